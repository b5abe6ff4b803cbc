// Forest / fern backward: dX, dThresholds, dWeights.
//
// Global floating-point atomics are far too slow for the 10^8..10^9 updates of a large batch, so every gradient is
// accumulated on chip and written once. The pass is a short pipeline over "walk records":
//
//   records   tile kernel (the forward's walk): per (tree, sample) the leaf key, the selected vertex, its ordinal and
//             the signed margin, stored tree major.
//   trees     tree-stationary: a workgroup owns a group of adjacent trees whose dW accumulators fill its LDS, streams
//             all samples once (one thread per sample; the group's slice of the upstream gradient row is contiguous),
//             adds |margin| * g into the LDS accumulators, and forms c = sign(margin) * sum_m w[t,leaf,m] * g[m],
//             which it stores tree major. dW is written from LDS at the end (plain stores; atomics only if the
//             samples had to be split over several workgroups).
//   dthr      tree-stationary: per tree, -c is accumulated by selected vertex in LDS.
//   dx        sample-stationary: a workgroup owns a tile of samples and a [features x tile] accumulator in LDS, adds
//             each tree's c at the selected ordinal, and writes the tile of dX once.
//
// Deterministic mode reuses the records and replaces the three accumulating kernels by owner-computes kernels whose
// order of additions is fixed (see below). Small problems, very deep trees and very wide inputs use a single fused
// kernel with global atomics instead.
#include <type_traits>

#include "forest_tile.hpp"
#include "lds_accumulate.hpp"
#include "records.hpp"

namespace ht {
namespace {

constexpr int kIlp = 4;         // trees walked concurrently per thread by the records kernel

// ---------------------------------------------------------------------------------------------------------------
// walk records (layout in records.hpp)
// ---------------------------------------------------------------------------------------------------------------
template <typename Real, bool FERN, int BT, bool XLDS, bool COMPACT>
__global__ __launch_bounds__(kForestThreads) void records_kernel(ForestDims d, const Real *__restrict__ x,
                                                                 const Node<Real> *__restrict__ nodes,
                                                                 Records<Real, COMPACT> rec, int trees_per_block) {
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
  const bool live = s < d.S;  // (dead lanes stay for the wavefront-wide publication of the margin bound)
  const long long xbase = live ? (s / d.K) * d.FK + (s % d.K) : 0;
  const int t_begin = blockIdx.y * trees_per_block;
  const int t_end = min(d.T, t_begin + trees_per_block);
  MarginBits margin_bound;
  for (int tb = t_begin + tt; live && tb < t_end; tb += TC * kIlp) {
    const Node<Real> *nd[kIlp];
    int t[kIlp];
#pragma unroll
    for (int i = 0; i < kIlp; ++i) {
      t[i] = tb + i * TC;
      nd[i] = nodes + (long long)min(t[i], t_end - 1) * d.V;
    }
    WalkResult<Real> r[kIlp];
    if (XLDS)
      walk_many<Real, FERN, kIlp>(d.depth, nd, [&](int, int f) { return xs[f * BT + j]; }, r);
    else
      walk_many<Real, FERN, kIlp>(d.depth, nd, [&](int, int f) { return x[xbase + (long long)f * d.K]; }, r);
#pragma unroll
    for (int i = 0; i < kIlp; ++i)
      if (t[i] < t_end) {
        rec.put((long long)t[i] * d.S + s, r[i].key, r[i].vertex, r[i].ord, r[i].margin);
        margin_bound.take(r[i].margin);
      }
  }
  bound_publish(margin_bound_value<Real>(margin_bound.bits), rec.bound, (blockIdx.y * gridDim.x + blockIdx.x) % unsigned(kBoundSlots));
}

template <typename Real, bool FERN, int BT, bool XLDS, bool COMPACT>
int launch_records(const ForestDims &d, const Real *x, const Node<Real> *nodes, Records<Real, COMPACT> rec,
                   hipStream_t stream) {
  constexpr int TP = kForestThreads / BT * kIlp;
  const size_t lds = XLDS ? size_t(d.F) * BT * sizeof(Real) : 0;
  const long long tiles = (d.S + BT - 1) / BT;
  int trees_per_block, gy;
  split_trees(tiles, d.T, TP, &trees_per_block, &gy);
  if (tiles > 0x7fffffffLL) return fail(HT_ERR_RUNTIME, "Error: too many sample tiles for one launch.");
  auto kernel = records_kernel<Real, FERN, BT, XLDS, COMPACT>;
  HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));
  hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)gy), dim3(kForestThreads), lds, stream, d, x, nodes, rec,
                     trees_per_block);
  HT_LAUNCH_CHECK("forest walk records");
  return HT_OK;
}

template <typename Real, bool FERN, bool COMPACT>
int dispatch_records(const ForestDims &d, const Real *x, const Node<Real> *nodes, Records<Real, COMPACT> rec,
                     hipStream_t stream) {
  switch (pick_tile<Real>(d.F, 1024)) {
    case 64: return launch_records<Real, FERN, 64, true, COMPACT>(d, x, nodes, rec, stream);
    case 32: return launch_records<Real, FERN, 32, true, COMPACT>(d, x, nodes, rec, stream);
    case 16: return launch_records<Real, FERN, 16, true, COMPACT>(d, x, nodes, rec, stream);
    case 8: return launch_records<Real, FERN, 8, true, COMPACT>(d, x, nodes, rec, stream);
    default: return launch_records<Real, FERN, 64, false, COMPACT>(d, x, nodes, rec, stream);
  }
}

// ---------------------------------------------------------------------------------------------------------------
// fixed-point accumulation (deterministic mode)
// ---------------------------------------------------------------------------------------------------------------
// Integer addition is associative, so sums kept as 64-bit integers do not depend on the order in which the hardware
// applies the atomics: the accumulating kernels below run unchanged, massively parallel, and are still bit
// reproducible. Each term is scaled by a power of two 2^k and rounded to an integer once; k is chosen on the device from
// a bound on the largest term and the largest number of terms a cell can receive so that no sum can overflow:
//   dW terms   |margin| * g   bound max|margin| * max|g|, at most S terms per cell
//   dThr / dX  c              bound max|c| (measured),    at most max(S, T) terms per cell
// which leaves >= 61 - ceil(log2(count)) bits below the largest term (an fp32 running sum keeps 24). Non-finite
// bounds (inf / NaN in the inputs) cannot be represented: the header then routes the affected gradients to the
// sequential owner-computes kernels further down, on the device, without a host round trip.
//
// Sampled bound (large upstream gradients on the lean tree kernel). A pass over the whole upstream gradient just for
// max|g| costs half as much again as the tree kernel that follows it. So max|g| is taken over a fixed 1/64 sample
// (whole 1 KB runs, their position inside each 64 KB advancing from run to run so that every column is met), the
// scale is chosen kSampleGuard times more generous than that sample asks for (10 of the spare bits), and the tree
// kernel, which sees every term anyway, keeps the largest |term| it accumulated. A check kernel then compares: if no
// term exceeded what the scale allows, the sums are exact sums of correctly rounded terms and stand; otherwise (a
// gradient with outliers more than kSampleGuard times the sample's largest value, or zero wherever it was sampled) the
// scale is chosen again from the true largest term and the tree kernel runs a second time -- all decided on the device
// and by the data alone, so the result stays bit reproducible.
struct DetHeader {
  unsigned long long max_g, max_a, max_c;  // bit patterns of non-negative doubles (ordered like the values)
  double scale_w, inv_scale_w, scale_c, inv_scale_c;
  int fallback_w, fallback_c;
  int redo_w;  // sampled bound exceeded: the second run of the tree kernel is wanted
};
constexpr double kSampleGuard = 1024.0;
constexpr int kSampleEvery = 64;                       // one run in 64 is read
constexpr size_t kSampleMinBytes = size_t(64) << 20;   // below that the full pass costs a few microseconds
// The bound on |c| is taken by the tree kernels as they store c (one running maximum per lane, one atomic per
// wavefront): the atomics go to kDetSlots slots behind the header, spread by workgroup, because thousands of atomics
// on ONE address serialise in L2 for longer than a pass over c takes; the scale kernel folds the slots.
// A second set of slots takes the largest |term| of dW the same way, a third the sample of max|g| (sampled bound).
constexpr int kDetSlots = 4096;
constexpr int kDetFoldThreads = 1024;
constexpr size_t kDetHeaderBytes = 256 + 3 * size_t(kDetSlots) * sizeof(unsigned long long);
__device__ __forceinline__ unsigned long long *det_slots(DetHeader *h) {
  return reinterpret_cast<unsigned long long *>(reinterpret_cast<unsigned char *>(h) + 256);
}
__device__ __forceinline__ unsigned long long *det_term_slots(DetHeader *h) { return det_slots(h) + kDetSlots; }
__device__ __forceinline__ unsigned long long *det_g_slots(DetHeader *h) { return det_slots(h) + 2 * kDetSlots; }

// Largest of n slots (bit patterns of non-negative doubles order like the values), by a workgroup of kDetFoldThreads
// threads; every thread receives it.
__device__ inline unsigned long long det_fold(const unsigned long long *slots, int n) {
  __shared__ unsigned long long part[kDetFoldThreads / kWave];
  unsigned long long m = 0ull;
  for (int i = threadIdx.x; i < n; i += kDetFoldThreads) m = max(m, slots[i]);
  for (int off = 32; off > 0; off >>= 1) m = max(m, (unsigned long long)__shfl_xor((long long)m, off, kWave));
  __syncthreads();  // a previous fold's readers are done with part[]
  if ((threadIdx.x & (kWave - 1)) == 0) part[threadIdx.x / kWave] = m;
  __syncthreads();
  m = 0ull;
  for (int i = 0; i < kDetFoldThreads / kWave; ++i) m = max(m, part[i]);
  return m;
}

__global__ __launch_bounds__(256) void det_init_kernel(DetHeader *h) {
  if (threadIdx.x == 0) {
    h->max_g = h->max_a = h->max_c = 0ull;
    h->scale_w = h->inv_scale_w = h->scale_c = h->inv_scale_c = 1.0;
    h->fallback_w = h->fallback_c = h->redo_w = 0;
  }
  for (int i = threadIdx.x; i < 3 * kDetSlots; i += 256) det_slots(h)[i] = 0ull;
}

// A lane's bound on |c| (bound_take, records.hpp) over the wavefront into the workgroup's slot.
template <typename Real>
__device__ __forceinline__ void publish_c_bound(Real m, const DetHeader *hdr) {
  bound_publish(double(m), det_slots(const_cast<DetHeader *>(hdr)),
                (blockIdx.y * gridDim.x + blockIdx.x) % unsigned(kDetSlots));
}
// A lane's bound on the |term| it added to dW (MarginBits, records.hpp), likewise.
__device__ __forceinline__ void publish_term_bound(MarginBits m, const DetHeader *hdr) {
  bound_publish(margin_bound_value<float>(m.bits), det_term_slots(const_cast<DetHeader *>(hdr)),
                (blockIdx.y * gridDim.x + blockIdx.x) % unsigned(kDetSlots));
}

// max |p[i]| (NaN counts as +inf) folded into *slot. A grid-stride loop of plain 16-byte loads, one in flight per
// thread: with 2048 workgroups of 512 threads that is the form in which a read stream runs fastest here (6.4 TB/s
// measured; four loads in flight per thread gave 5.4).
constexpr int kAbsmaxThreads = 512;
template <typename Real>
__global__ __launch_bounds__(kAbsmaxThreads) void absmax_kernel(const Real *__restrict__ p, long long n,
                                                                unsigned long long *slot) {
  constexpr int VEC = 16 / sizeof(Real);
  typedef Real Vec __attribute__((ext_vector_type(VEC)));
  Real m = Real(0);
  const long long tid = (long long)blockIdx.x * kAbsmaxThreads + threadIdx.x;
  const long long nthreads = (long long)gridDim.x * kAbsmaxThreads;
  long long body = 0;
  if (reinterpret_cast<uintptr_t>(p) % 16 == 0) {
    body = n / VEC;
    const Vec *pv = reinterpret_cast<const Vec *>(p);
    for (long long i = tid; i < body; i += nthreads) {
      const Vec v = pv[i];
#pragma unroll
      for (int e = 0; e < VEC; ++e) bound_take(m, v[e]);
    }
    body *= VEC;
  }
  for (long long i = body + tid; i < n; i += nthreads) bound_take(m, p[i]);
  double md = double(m);
  for (int off = 32; off > 0; off >>= 1) {
    const double o = __shfl_xor(md, off, kWave);
    if (!(o <= md)) md = o;
  }
  // one atomic per workgroup: thousands of atomics on the one slot would serialise in L2 for longer than the pass reads
  __shared__ double part[kAbsmaxThreads / kWave];
  if ((threadIdx.x & (kWave - 1)) == 0) part[threadIdx.x / kWave] = md;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int i = 1; i < kAbsmaxThreads / kWave; ++i)
      if (!(part[i] <= md)) md = part[i];
    if (md > 0.0) atomicMax(slot, (unsigned long long)__double_as_longlong(md));
  }
}

// The same over a sample: of every kSampleEvery consecutive 1 KB runs (64 x 16 bytes, one load of a wavefront) one is
// read, run k of the sample at position (37 k mod kSampleEvery) of its 64 KB, so that the sample meets every column of
// any row length. p is 16-byte aligned.
template <typename Real>
__global__ __launch_bounds__(kAbsmaxThreads) void absmax_sample_kernel(const Real *__restrict__ p, long long runs,
                                                                       unsigned long long *slots) {
  constexpr int VEC = 16 / sizeof(Real);
  typedef Real Vec __attribute__((ext_vector_type(VEC)));
  const Vec *pv = reinterpret_cast<const Vec *>(p);
  const int lane = threadIdx.x & (kWave - 1);
  const long long wave = ((long long)blockIdx.x * kAbsmaxThreads + threadIdx.x) / kWave;
  const long long waves = (long long)gridDim.x * (kAbsmaxThreads / kWave);
  Real m = Real(0);
  for (long long k = wave; k < runs; k += waves) {
    const long long run = k * kSampleEvery + ((k * 37) & (kSampleEvery - 1));
    const Vec v = pv[run * kWave + lane];
#pragma unroll
    for (int e = 0; e < VEC; ++e) bound_take(m, v[e]);
  }
  double md = double(m);
  for (int off = 32; off > 0; off >>= 1) {
    const double o = __shfl_xor(md, off, kWave);
    if (!(o <= md)) md = o;
  }
  __shared__ double part[kAbsmaxThreads / kWave];
  if (lane == 0) part[threadIdx.x / kWave] = md;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int i = 1; i < kAbsmaxThreads / kWave; ++i)
      if (!(part[i] <= md)) md = part[i];
    if (md > 0.0) atomicMax(slots + blockIdx.x % unsigned(kDetSlots), (unsigned long long)__double_as_longlong(md));
  }
}

__device__ inline void det_pick_scale(double bound, double count, double *scale, double *inv, int *fallback) {
  if (!(bound < double(INFINITY))) {
    *fallback = 1;
    *scale = *inv = 0.0;
    return;
  }
  *fallback = 0;
  if (bound == 0.0) {
    *scale = *inv = 1.0;
    return;
  }
  int e;
  frexp(bound, &e);  // bound < 2^e
  int bits = 0;
  while (ldexp(1.0, bits) < count) ++bits;
  // a product rounded to Real can exceed the bound by an ulp: 61, not 62, keeps every sum inside int64; and a single
  // term stays below 2^50 whatever the count (to_fixed)
  int k = 61 - e - bits;
  if (k > 50 - e) k = 50 - e;
  k = k > 1000 ? 1000 : (k < -1000 ? -1000 : k);
  *scale = ldexp(1.0, k);
  *inv = ldexp(1.0, -k);
}

// which = 0: scale of dW from max|g| (measured by a full pass, or folded here from the sample's slots) x max|margin|
// (folded from the slots that came with the records) x guard; which = 1: scale of dThr / dX from max|c| (folded from
// the slots the tree kernel filled).
__global__ __launch_bounds__(kDetFoldThreads) void det_scale_kernel(DetHeader *h, int which, double count,
                                                                    bool fold_slots,
                                                                    const unsigned long long *margin_slots,
                                                                    double guard, bool sampled) {
  if (which == 0) {
    const unsigned long long a = margin_slots ? det_fold(margin_slots, kBoundSlots) : 0ull;
    const unsigned long long g = sampled ? det_fold(det_g_slots(h), kDetSlots) : 0ull;
    if (threadIdx.x == 0) {
      if (margin_slots) h->max_a = a;
      if (sampled) h->max_g = g;
    }
  }
  if (which == 1 && fold_slots) {
    const unsigned long long c = det_fold(det_slots(h), kDetSlots);
    if (threadIdx.x == 0) h->max_c = c;
  }
  if (threadIdx.x != 0) return;
  if (which == 0)
    det_pick_scale(guard * __longlong_as_double((long long)h->max_g) * __longlong_as_double((long long)h->max_a),
                   count, &h->scale_w, &h->inv_scale_w, &h->fallback_w);
  else
    det_pick_scale(__longlong_as_double((long long)h->max_c), count, &h->scale_c, &h->inv_scale_c, &h->fallback_c);
}

// Sampled bound: did every term the tree kernel accumulated stay inside what the scale of dW was chosen for? If not,
// the scale is chosen again from the true largest term and the second run of the tree kernel is switched on (a
// non-finite term routes dW to the sequential kernel instead, like a non-finite bound does).
__global__ __launch_bounds__(kDetFoldThreads) void det_verify_kernel(DetHeader *h, double count, double guard) {
  const unsigned long long m = det_fold(det_term_slots(h), kDetSlots);
  if (threadIdx.x != 0 || h->fallback_w) return;
  const double largest = __longlong_as_double((long long)m);
  const double allowed = guard * __longlong_as_double((long long)h->max_g) * __longlong_as_double((long long)h->max_a);
  if (largest <= allowed) return;
  det_pick_scale(largest, count, &h->scale_w, &h->inv_scale_w, &h->fallback_w);
  h->redo_w = h->fallback_w ? 0 : 1;
}

// Clears n 64-bit words if *flag is set.
__global__ __launch_bounds__(256) void zero_if_kernel(unsigned long long *p, long long n, const int *flag) {
  if (!*flag) return;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) p[i] = 0ull;
}

// round(v * scale) as a 64-bit integer, for |v * scale| < 2^51 (det_pick_scale keeps every term below 2^50): adding
// 1.5 * 2^52 leaves the rounded integer, as a two's complement offset, in the low bits of the double -- one fused
// multiply-add and one 64-bit subtraction where a conversion instruction sequence takes a dozen; same rounding (to
// nearest, ties to even). Larger products (a sampled bound that did not hold: the run is repeated) give some integer.
__device__ __forceinline__ unsigned long long to_fixed(double v, double scale) {
  return (unsigned long long)(__double_as_longlong(__builtin_fma(v, scale, 0x1.8p52)) - 0x4338000000000000LL);
}
template <typename Real>
__device__ __forceinline__ Real from_fixed(unsigned long long q, double inv) {
  return Real(double((long long)q) * inv);
}

// out[i] = fixed[i] / scale (skipped when the header routed this gradient to the sequential kernels).
template <typename Real>
__global__ __launch_bounds__(256) void fixed_to_real_kernel(const unsigned long long *__restrict__ src, Real *dst,
                                                            long long n, const DetHeader *h, int which) {
  if (which == 0 ? h->fallback_w : h->fallback_c) return;
  const double inv = which == 0 ? h->inv_scale_w : h->inv_scale_c;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256)
    dst[i] = from_fixed<Real>(src[i], inv);
}

// ---------------------------------------------------------------------------------------------------------------
// tree-stationary dW + c
// ---------------------------------------------------------------------------------------------------------------
// grid = (tree groups, sample parts). Workgroup (g, p) owns trees [g*TB, g*TB + nt) and the samples of part p.
// LDS: dW accumulators [nt][L][M] in fp64 (if dw): the fp64 LDS atomic add is a fast hardware instruction on gfx950,
// the fp32 one is not (see lds_accumulate.hpp); each product |margin| * g is still rounded to Real first, only the
// running sum is wider.
//
// The kernel is bound by the number of accesses its loads cost in the vector memory pipeline, which handles a load
// four lanes at a time and charges every distinct line those four lanes touch. So:
//   * records are loaded one pair per lane, trees in lane blocks (lanes [r*SPT, r*SPT + SPT) hold SPT consecutive
//     samples of tree r): fully coalesced, one load per 64 pairs; c is stored the same way.
//   * a pair's M upstream-gradient values and its M leaf weights are each one contiguous run of memory. It is read by
//     P adjacent lanes (P a power of two, so groups never straddle a quad unless they fill several) with one 16-byte
//     load per lane; the last lane's chunk is shifted back to end at M, and it owns only the elements past its
//     neighbour's. Pairs are taken sample major, tree minor, so adjacent lane groups read adjacent memory.
//   * the record fields travel from the lane that loaded them to the lanes that need them by ds_bpermute.
//
// FIXED (deterministic mode): the accumulators are 64-bit fixed point (see above); partial sums of sample parts are
// merged with integer atomics into dw_fixed and converted by fixed_to_real_kernel.
constexpr int kMaxGroupTrees = 16;

// Tree group of workgroup column x (a grid row has 8 * ceil(groups / 8) columns), or -1 for a surplus column.
// Workgroups are dealt to the 8 XCDs round robin by index and each XCD has its own L2; adjacent tree groups read
// adjacent pieces of the same 128-byte lines of the upstream gradient, so they are placed on the same XCD (group =
// (index mod 8) * groups_per_xcd + index / 8): the line is then fetched from memory once instead of once per XCD.
__device__ __forceinline__ int xcd_tree_group(unsigned x, int num_groups) {
  const int per_xcd = (num_groups + kNumXCDs - 1) / kNumXCDs;
  const int group = int(x % kNumXCDs) * per_xcd + int(x / kNumXCDs);
  return group < num_groups ? group : -1;
}

template <int CTRL>
__device__ __forceinline__ float dpp_swap(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ double dpp_swap(double v) {
  const int lo = __builtin_amdgcn_update_dpp(0, __double2loint(v), CTRL, 0xF, 0xF, true);
  const int hi = __builtin_amdgcn_update_dpp(0, __double2hiint(v), CTRL, 0xF, 0xF, true);
  return __hiloint2double(hi, lo);
}
// Sum over aligned groups of P adjacent lanes (P a power of two); every lane of a group receives the total.
template <typename Real>
__device__ __forceinline__ Real group_sum(Real v, int P) {
  if (P >= 2) v += dpp_swap<0xB1>(v);  // quad_perm [1,0,3,2]
  if (P >= 4) v += dpp_swap<0x4E>(v);  // quad_perm [2,3,0,1]
  for (int off = 4; off < P; off <<= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

template <typename Real, bool COMPACT, bool FIXED, int U>
__global__ __launch_bounds__(kForestThreads) void tree_kernel(ForestDims d, const Real *__restrict__ w,
                                                              const Real *__restrict__ gout,
                                                              Records<Real, COMPACT> rec, Real *dw,
                                                              unsigned long long *dw_fixed, const DetHeader *hdr,
                                                              int TB, long long part_size, bool need_c,
                                                              bool dw_atomic, int P, int num_groups, int slices,
                                                              int m0, int Mw) {
  // [m0, m0 + Mw): the window of a leaf row's elements this launch serves. A row wider than the 64 lanes x 16 bytes a
  // wavefront can give one pair is worked off in several launches, each with accumulators for its window only; c,
  // a sum over the whole row, is then built up launch by launch.
  constexpr int VE = 16 / sizeof(Real);  // elements per 16-byte chunk
  typedef typename std::conditional<FIXED, unsigned long long, double>::type Acc;
  extern __shared__ __align__(16) unsigned char smem[];
  Acc *acc = reinterpret_cast<Acc *>(smem);
  double scale = 1.0, inv_scale = 1.0;
  if (FIXED) {
    if (hdr->fallback_w) dw = nullptr;
    scale = hdr->scale_w;
    inv_scale = hdr->inv_scale_w;
    if (!dw && !need_c) return;
  }
  int group = xcd_tree_group(blockIdx.x, num_groups);
  if (group < 0) return;
  // slices > 1 (one tree per group; its leaf table does not fit LDS): `slices` consecutive groups serve the same tree,
  // each accumulating the leaves [leaf_begin, leaf_begin + leaves) only. Every slice streams all records and gradient
  // rows of the tree (the loads go out before the keys are known; loading a slice's own rows only, once the keys are
  // there, was measured slower: the chain record -> row costs more than the L2 traffic it saves); c is computed by
  // the first slice.
  const int slice = group % slices;
  group /= slices;
  const int leaves = d.L / slices;
  const uint32_t leaf_begin = uint32_t(slice) * uint32_t(leaves);
  if (slice != 0) need_c = false;
  if (!dw && !need_c) return;
  const int t0 = group * TB;
  const int nt = min(TB, d.T - t0);
  const long long LM = (long long)d.L * d.M;
  const long long acc_cells = (long long)nt * leaves * Mw;  // (nt == 1 whenever slices > 1)
  if (dw) {
    for (long long i = threadIdx.x; i < acc_cells; i += kForestThreads) acc[i] = Acc(0);
    __syncthreads();
  }
  const long long s_begin = (long long)blockIdx.y * part_size;
  const long long s_end = min(d.S, s_begin + part_size);
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  constexpr int kWaves = kForestThreads / kWave;
  const int SPT = kWave / nt;  // samples per tree in one 64-pair block
  const int NP = kWave / P;    // pairs per sub-step; a block has P sub-steps, taken U at a time (U divides P)
  const FastDiv div_nt(nt), div_spt(SPT);

  // this lane as a loader of records: tree rt, sample offset rj of the block
  const int rt = div_spt.div(lane), rj = lane - rt * SPT;
  const bool rec_lane = rt < nt;
  // ... and where that pair is processed: sub-step my_sub, lane group my_src / P
  const int my_pp = rj * nt + rt;
  const int my_sub = my_pp / NP, my_src = (my_pp - my_sub * NP) * P;
  // this lane as a member of a lane group.
  // The M elements are dealt evenly to the P lanes (lane li owns [li*M/P, (li+1)*M/P): at least one, at most VE), so
  // the LDS atomics -- whose cost is per instruction, not per active lane -- need only ceil(M/P) rounds. A lane loads
  // the 16-byte chunk that starts at its first element (shifted back where it would pass the end of the row): lanes
  // with overlapping chunks hit the same line, which costs nothing extra.
  const int grp = lane / P, li = lane & (P - 1);
  const int own_begin = li * Mw / P, own_end = (li + 1) * Mw / P;  // inside the window
  const int e0 = Mw >= VE ? min(own_begin, Mw - VE) : 0;  // first element of this lane's chunk
  const int own = own_begin - e0;                          // chunk elements [own, own + cnt) belong to this lane
  const int cnt = own_end - own_begin;
  const int rounds = (Mw + P - 1) / P;                     // wave uniform: max cnt over the lanes

  auto load_chunk = [&](const Real *p, Real (&v)[VE]) {
    if (Mw >= VE) {
      __builtin_memcpy(v, p, sizeof(Real) * VE);  // 16 bytes, element aligned
    } else {
#pragma unroll
      for (int k = 0; k < VE; ++k) v[k] = k < Mw ? p[k] : Real(0);
    }
  };

  // The samples of a wavefront form blocks of SPT (x nt trees = up to 64 pairs); a block is worked off in P / U
  // chunks of U sub-steps. Per chunk the record loads and the gradient loads (whose addresses depend on nothing
  // loaded) go out together; the weight loads follow when the keys are there. Every load is unconditional, idle lanes
  // aimed at the block's first pair, which keeps the number of loads in flight at each wait a compile-time constant,
  // so a wait never covers more than it has to. (Prefetching the next chunk during the arithmetic was measured and
  // did not pay: the kernel is not latency bound.)
  struct Chunk {
    long long at;   // record index of this lane as a loader
    bool have;      // ... and whether it holds a pair
    int npairs;
    uint32_t key_r;
    Real mg_r;
    bool on[U];
    int src[U], tq_of[U];
    Real gv[U][VE];
  };
  const Real *wbase = w + (long long)t0 * LM;
  const int CPB = P / U;  // chunks per block (a power of two)
  const long long my_first = s_begin + (long long)wave * SPT;
  const long long nblk = my_first < s_end ? (s_end - my_first + (long long)kWaves * SPT - 1) / ((long long)kWaves * SPT) : 0;
  const long long nchunks = nblk * CPB;

  auto prefetch = [&](long long c, Chunk &q) {
    const long long blk = c / CPB;
    const int sub0 = int(c - blk * CPB) * U;
    const long long sblk = my_first + blk * kWaves * SPT;
    const int ns = int(min<long long>(SPT, s_end - sblk));
    q.npairs = ns * nt;
    q.have = rec_lane && rj < ns;
    q.at = (long long)(t0 + (q.have ? rt : 0)) * d.S + sblk + (q.have ? rj : 0);
    q.key_r = rec.key(q.at);
    q.mg_r = rec.margin[q.at];
    const Real *gbase = gout + (d.K == 1 ? (sblk * d.T + t0) * d.M : 0);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int pp = (sub0 + u) * NP + grp;
      q.on[u] = pp < q.npairs;
      const int j = q.on[u] ? div_nt.div(pp) : 0;
      const int tq = q.on[u] ? pp - j * nt : 0;
      q.src[u] = tq * SPT + j;
      q.tq_of[u] = tq;
      if (d.K == 1)
        load_chunk(gbase + (uint32_t(j) * d.T + tq) * d.M + m0 + e0, q.gv[u]);
      else
        load_chunk(gout + out_offset(d, sblk + j, t0 + tq, m0 + e0), q.gv[u]);
    }
  };

  Real c_mine = Real(0), c_bound = Real(0);
  for (long long c = 0; c < nchunks; ++c) {
    const int sub0 = int(c & (CPB - 1)) * U;
    Chunk cur;
    prefetch(c, cur);
    uint32_t rel[U];
    bool in_slice[U];
    Real mg[U];
    Real wv[U][VE];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t key = __shfl(cur.key_r, cur.src[u], kWave);
      mg[u] = __shfl(cur.mg_r, cur.src[u], kWave);
      const uint32_t row = uint32_t(cur.tq_of[u]) * d.L + key;
      if (need_c) load_chunk(wbase + (row * uint32_t(d.M) + uint32_t(m0) + e0), wv[u]);
      // the pair's accumulator row: this slice's leaves only, counted from the slice's first leaf; the window's
      // elements only
      in_slice[u] = cur.on[u] && key - leaf_begin < uint32_t(leaves);
      rel[u] = (row - leaf_begin) * uint32_t(Mw) + e0;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (dw && in_slice[u]) {
        const Real a = ht_abs(mg[u]);
        Acc *cell = acc + rel[u];
#pragma unroll
        for (int i = 0; i < VE; ++i) {
          if (i >= rounds) break;  // wave uniform
          if (i < cnt) {
            // element own + i of the chunk (own is not a compile-time constant: select, do not index)
            Real g = cur.gv[u][0];
#pragma unroll
            for (int k = 1; k < VE; ++k) g = (own + i == k) ? cur.gv[u][k] : g;
            if (FIXED)
              atomicAdd(reinterpret_cast<unsigned long long *>(cell) + own + i, to_fixed(double(a * g), scale));
            else
              atomicAdd(reinterpret_cast<double *>(cell) + own + i, double(a * g));
          }
        }
      }
      if (need_c) {
        Real partial = Real(0);
#pragma unroll
        for (int k = 0; k < VE; ++k)
          if (k >= own && k < own + cnt) partial += wv[u][k] * cur.gv[u][k];
        partial = group_sum<Real>(cur.on[u] ? partial : Real(0), P);
        const Real got = __shfl(ht_sign(mg[u]) * partial, my_src, kWave);
        if (my_sub == sub0 + u) c_mine = got;
      }
    }
    if (need_c && sub0 + U == P && cur.have) {
      if (m0 != 0) c_mine += rec.c[cur.at];  // the earlier windows' share (the launches follow each other)
      rec.c[cur.at] = c_mine;
      if (FIXED) bound_take(c_bound, c_mine);
    }
  }
  if (FIXED && need_c) publish_c_bound(c_bound, hdr);
  if (dw) {
    __syncthreads();
    const long long first = (long long)t0 * LM + (long long)leaf_begin * d.M + m0;
    Real *dst = dw + first;
    // cell i of the table is element i % Mw of accumulator row i / Mw: where it lies in a row of d.M elements
    const FastDiv by_mw(Mw);
    auto at = [&](long long i) -> long long {
      if (Mw == d.M) return i;
      const long long row = acc_cells < (1ll << 31) ? (long long)by_mw.div(int(i)) : i / Mw;
      return row * d.M + (i - row * Mw);
    };
    if (FIXED) {
      const unsigned long long *q = reinterpret_cast<const unsigned long long *>(acc);
      if (dw_atomic) {
        for (long long i = threadIdx.x; i < acc_cells; i += kForestThreads)
          if (q[i] != 0ull) atomicAdd(dw_fixed + first + at(i), q[i]);
      } else {
        for (long long i = threadIdx.x; i < acc_cells; i += kForestThreads) dst[at(i)] = from_fixed<Real>(q[i], inv_scale);
      }
    } else {
      const double *q = reinterpret_cast<const double *>(acc);
      if (dw_atomic) {
        for (long long i = threadIdx.x; i < acc_cells; i += kForestThreads)
          if (q[i] != 0.0) atomicAdd(dst + at(i), Real(q[i]));
      } else {
        for (long long i = threadIdx.x; i < acc_cells; i += kForestThreads) dst[at(i)] = Real(q[i]);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// tree-stationary dW + c, specialised: float, K == 1, compact records, M a compile-time constant, TB a power of two
// ---------------------------------------------------------------------------------------------------------------
// Same work split as tree_kernel; what differs is that everything that does not depend on the data (which lane
// serves which pair, every address offset, which chunk elements a lane owns) is computed once per lane outside the
// sample loop, M / P are compile-time constants, and a lane group finds its records inside its own quad, so a 64-pair
// block costs a fraction of the generic kernel's vector and LDS instructions -- the generic kernel is bound by
// instruction issue and by the LDS pipeline (atomics + cross-lane permutes), not by memory.
//
// A block is SPT = 64 / TB consecutive samples x TB trees = 64 pairs. It is worked off in P sub-steps of 64 / P
// pairs; lane li = lane % P of a lane group owns CNT(li) of a pair's M elements and loads the 16-byte chunk that
// starts at its first element, except that the last lane's chunk is the row's last four elements. A record reaches
// the lanes of its group through a DPP quad broadcast (a plain vector instruction) instead of an LDS permute.
template <int M>
struct LeanSplit {
  static constexpr int VE = 4;
  static constexpr int Q = (M + VE - 1) / VE;
  static constexpr int P = Q <= 1 ? 1 : (Q <= 2 ? 2 : 4);  // lanes per pair (M <= 16)
  static constexpr int BASE = M / P, EXTRA = M % P;         // lanes li < EXTRA own BASE + 1 elements
  static constexpr int ROUNDS = BASE + (EXTRA ? 1 : 0);
  static constexpr int LAST = M >= VE ? M - VE : 0;         // first element of the row's last chunk
  __host__ __device__ static constexpr int begin(int li) { return li * BASE + (li < EXTRA ? li : EXTRA); }
  __host__ __device__ static constexpr int count(int li) { return BASE + (li < EXTRA ? 1 : 0); }
  // chunk position of the last lane's first own element
  static constexpr int SHIFT = (M >= VE && begin(P - 1) > LAST) ? begin(P - 1) - LAST : 0;
};

typedef float Float4U __attribute__((ext_vector_type(4), aligned(4)));

template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

// Value of lane (group base + U) of each aligned group of P lanes (P <= 4), to every lane of the group.
template <int P, int U>
__device__ __forceinline__ int group_bcast(int v) {
  if constexpr (P == 1) {
    return v;
  } else if constexpr (P == 2) {
    constexpr int ctrl = U | (U << 2) | ((2 + U) << 4) | ((2 + U) << 6);  // quad_perm [U, U, 2+U, 2+U]
    return __builtin_amdgcn_update_dpp(0, v, ctrl, 0xF, 0xF, true);
  } else {
    constexpr int ctrl = U * 0x55;  // quad_perm [U, U, U, U]
    return __builtin_amdgcn_update_dpp(0, v, ctrl, 0xF, 0xF, true);
  }
}

template <int M, bool FIXED, bool WLDS>
__global__ __launch_bounds__(kForestThreads) void tree_lean_kernel(ForestDims d, const float *__restrict__ w,
                                                                   const float *__restrict__ gout,
                                                                   Records<float, true> rec, float *dw,
                                                                   unsigned long long *dw_fixed,
                                                                   const DetHeader *hdr, int log2_tb,
                                                                   long long part_size, bool need_c, bool dw_atomic,
                                                                   int num_groups, float *dthr_fold,
                                                                   uint32_t thr_lds_offset, uint32_t w_lds_offset,
                                                                   bool second_run) {
  static_assert(!WLDS || M == 1, "leaf weights are staged in LDS for single-output leaves only");
  typedef LeanSplit<M> Split;
  constexpr int P = Split::P, VE = Split::VE, ROUNDS = Split::ROUNDS, SHIFT = Split::SHIFT;
  static_assert(M <= 16, "at most four lanes per pair");
  static_assert(M < VE || Split::begin(P - 1) + Split::count(P - 1) == M, "element split must cover the row");
  static_assert(M < VE || P < 2 || Split::begin(P - 2) <= Split::LAST, "only the last lane of a group is shifted");
  static_assert(SHIFT + Split::count(P - 1) <= VE, "the last lane's elements lie inside its chunk");
  typedef typename std::conditional<FIXED, unsigned long long, double>::type Acc;
  extern __shared__ __align__(16) unsigned char smem[];
  Acc *acc = reinterpret_cast<Acc *>(smem);
  // dthr_fold (atomic mode, where LDS has room behind the leaf accumulators): dThr of the group's trees is reduced
  // here as well, by selected vertex, and the separate pass over the records and c is not needed.
  double *acc_thr = reinterpret_cast<double *>(smem + thr_lds_offset);
  float *w_lds = reinterpret_cast<float *>(smem + w_lds_offset);  // WLDS: the group's leaf weights
  double scale = 1.0, inv_scale = 1.0;
  if (FIXED) {
    if (second_run && !hdr->redo_w) return;  // the sampled bound held (see DetHeader)
    if (hdr->fallback_w) dw = nullptr;
    scale = hdr->scale_w;
    inv_scale = hdr->inv_scale_w;
    if (!dw && !need_c) return;
  }
  MarginBits term_bound;  // FIXED: largest |term| this lane added to dW
  // A leaf's accumulators are M cells of 8 bytes. One atomic instruction touches the same element of different
  // leaves, so with M = 2^Z * odd its cells would fall on 32 / 2^Z of the LDS's 32 bank pairs only. The low Z bits of
  // a cell's index inside its row are therefore XORed with Z bits of the leaf key (bits that do not enter M * key
  // mod 32), which spreads them over all pairs; rows begin at multiples of 2^Z, so a cell stays inside its row. The
  // swizzle of a pair travels in the upper half of its `rel` word (offsets inside a group's table stay below 2^16
  // whenever the table exists).
  constexpr int Z = (M % 2) ? 0 : ((M % 4) ? 1 : ((M % 8) ? 2 : ((M % 16) ? 3 : 4)));
  constexpr uint32_t kSwizzleMask = (1u << Z) - 1u;
  auto swizzle_of = [&](uint32_t key) -> uint32_t { return Z == 0 ? 0u : (key >> (5 - Z)) & kSwizzleMask; };
  auto pack_rel = [&](uint32_t r, uint32_t key) -> uint32_t { return (Z != 0 && dw) ? (r | (swizzle_of(key) << 16)) : r; };
  const int TB = 1 << log2_tb;
  const int group = xcd_tree_group(blockIdx.x, num_groups);
  if (group < 0) return;
  const int t0 = group * TB;
  const int nt = min(TB, d.T - t0);
  const uint32_t LM = uint32_t(d.L) * M;
  if (dw)
    for (uint32_t i = threadIdx.x; i < uint32_t(nt) * LM; i += kForestThreads) acc[i] = Acc(0);
  if (dthr_fold)
    for (uint32_t i = threadIdx.x; i < uint32_t(nt) * uint32_t(d.V); i += kForestThreads) acc_thr[i] = 0.0;
  if (WLDS && need_c)
    for (uint32_t i = threadIdx.x; i < uint32_t(nt) * LM; i += kForestThreads) w_lds[i] = w[(long long)t0 * LM + i];
  if (dw || dthr_fold || WLDS) __syncthreads();
  const long long s_begin = (long long)blockIdx.y * part_size;
  const long long s_end = min(d.S, s_begin + part_size);
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  constexpr int kWaves = kForestThreads / kWave;
  const int SPT = kWave >> log2_tb;

  // ---- loop-invariant lane constants
  const int li = lane & (P - 1), grp = lane / P;
  const int my_begin = Split::begin(li), my_cnt = Split::count(li);
  const int e0 = M >= VE ? min(my_begin, Split::LAST) : 0;
  const bool shifted = SHIFT != 0 && li == P - 1;
  // Records are loaded one pair per lane, coalesced: lane = tree * SPT + sample. P divides SPT (TB <= 16), so the P
  // lanes of a group hold P consecutive samples of ONE tree, and those are the pairs the group serves in its P
  // sub-steps: sub-step u works on the pair whose record lane (group base + u) loaded.
  const int log2_spt = 6 - log2_tb;
  const int tq = lane >> log2_spt;                     // tree of this lane's group (and of its record)
  const int jq0 = (grp * P) & (SPT - 1);               // sample of the group's sub-step 0
  const int rec_t = tq, rec_j = jq0 + li;              // the pair whose record this lane loads and whose c it stores
  const uint32_t goff = (uint32_t(jq0) * uint32_t(d.T) + uint32_t(tq)) * M + e0;  // this lane's chunk, sub-step 0
  const uint32_t gstep = uint32_t(d.T) * M;                                        // ... and per further sub-step
  const uint32_t woff = uint32_t(tq) * LM + e0;  // (tree * L) * M + e0, to which key * M is added
  constexpr int jstep = 1;
  const float *wbase = w + (long long)t0 * LM;
  const uint32_t key_mask = rec.key_mask();

  // The ROUNDS elements this lane owns, out of a loaded chunk: positions 0.. for all lanes but the shifted one, which
  // takes SHIFT.. instead. The empty asm keeps the four components apart, so each own element costs one select with
  // a loop-invariant condition.
  auto own_elements = [&](Float4U v, float (&e)[ROUNDS]) {
    float c0 = v[0], c1 = v[1], c2 = v[2], c3 = v[3];
    if constexpr (SHIFT != 0) {
      asm volatile("" : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3));
      static_for<ROUNDS>([&](auto i_tag) {
        constexpr int i = decltype(i_tag)::value;
        constexpr int k = i + SHIFT < VE ? i + SHIFT : VE - 1;
        const float plain = i == 0 ? c0 : (i == 1 ? c1 : (i == 2 ? c2 : c3));
        const float moved = k == 0 ? c0 : (k == 1 ? c1 : (k == 2 ? c2 : c3));
        e[i] = shifted ? moved : plain;
      });
    } else {
      static_for<ROUNDS>([&](auto i_tag) {
        constexpr int i = decltype(i_tag)::value;
        e[i] = i == 0 ? c0 : (i == 1 ? c1 : (i == 2 ? c2 : c3));
      });
    }
  };
  auto load_chunk = [&](const float *p, bool stream) -> Float4U {
    Float4U v;
    if constexpr (M >= VE) {
      v = stream ? __builtin_nontemporal_load(reinterpret_cast<const Float4U *>(p))
                 : *reinterpret_cast<const Float4U *>(p);
    } else {
#pragma unroll
      for (int k = 0; k < VE; ++k) v[k] = k < M ? p[k] : 0.f;
    }
    return v;
  };

  // A block's state between the moment its loads are issued and the moment it is consumed.
  struct Stage {
    uint32_t a_r;   // record words of the pair this lane loads (key | vertex << 16, margin)
    float mg_r;
    float mg_own;   // copy of mg_r that survives the reuse of a_r / mg_r for a later block
    uint32_t v_own;  // ... and the selected vertex of that record
    float mg[P];    // per sub-step: margin of the pair this lane's group serves
    uint32_t rel[P];  // ... and its element offset (tree, leaf, first chunk element) in the group's weights
    Float4U gv[P], wv[P];
  };
  auto record_index = [&](long long sblk, bool have) -> long long {
    return (long long)(t0 + (have ? rec_t : 0)) * d.S + sblk + (have ? rec_j : 0);
  };
  auto issue_rec = [&](Stage &st, long long sblk, bool have) {
    const long long at = record_index(sblk, have);
    st.a_r = rec.a[at];
    st.mg_r = rec.margin[at];
  };
  auto issue_g = [&](Stage &st, long long sblk, const bool (&on)[P]) {
    const float *gbase = gout + (sblk * d.T + t0) * M;
#pragma unroll
    for (int u = 0; u < P; ++u) st.gv[u] = load_chunk(on[u] ? gbase + u * gstep + goff : gbase + e0, false);
  };
  auto issue_w = [&](Stage &st, const bool (&on)[P]) {
    st.mg_own = st.mg_r;
    if (dthr_fold) st.v_own = (st.a_r >> rec.vshift) & key_mask;
    static_for<P>([&](auto u_tag) {
      constexpr int u = decltype(u_tag)::value;
      const uint32_t key = uint32_t(group_bcast<P, u>(int(st.a_r))) & key_mask;
      st.mg[u] = __int_as_float(group_bcast<P, u>(__float_as_int(st.mg_r)));
      const uint32_t r = woff + key * M;
      st.rel[u] = pack_rel(r, key);
      if (need_c) {
        if constexpr (WLDS) {
          st.wv[u] = Float4U{w_lds[on[u] ? r : 0u], 0.f, 0.f, 0.f};
        } else {
          st.wv[u] = load_chunk(wbase + (on[u] ? r : uint32_t(e0)), false);
        }
      }
    });
  };
  float c_bound = 0.f;  // FIXED: largest |c| this lane stored
  auto compute = [&](Stage &st, long long sblk, bool have, const bool (&on)[P], auto full_tag) {
    constexpr bool FULL = decltype(full_tag)::value;
    float c_mine = 0.f;
#pragma unroll
    for (int u = 0; u < P; ++u) {
      float g[ROUNDS];
      own_elements(st.gv[u], g);
      if (dw && (FULL || on[u])) {
        const uint32_t row = (Z != 0 ? (st.rel[u] & 0xFFFFu) : st.rel[u]) - e0, swz = Z != 0 ? st.rel[u] >> 16 : 0u;
#pragma unroll
        for (int i = 0; i < ROUNDS; ++i) {
          if (i < Split::BASE || i < my_cnt) {
            const float term = ht_abs(st.mg[u]) * g[i];
            Acc *cell = acc + (row + ((uint32_t(my_begin) + i) ^ swz));
            if (FIXED) term_bound.take(term);
            if (FIXED)
              atomicAdd(reinterpret_cast<unsigned long long *>(cell), to_fixed(double(term), scale));
            else
              atomicAdd(reinterpret_cast<double *>(cell), double(term));
          }
        }
      }
      if (need_c) {
        float wl[ROUNDS];
        own_elements(st.wv[u], wl);
        float partial = 0.f;
#pragma unroll
        for (int i = 0; i < ROUNDS; ++i) {
          const float term = __builtin_fmaf(wl[i], g[i], partial);
          partial = (i < Split::BASE || i < my_cnt) ? term : partial;
        }
        partial = group_sum<float>((FULL || on[u]) ? partial : 0.f, P);
        c_mine = (li == u) ? partial : c_mine;
      }
    }
    if (need_c && (FULL || have)) {
      const float c = ht_sign(st.mg_own) * c_mine;
      rec.c[record_index(sblk, have)] = c;
      if (FIXED) bound_take(c_bound, c);
      if (dthr_fold) atomicAdd(acc_thr + uint32_t(rec_t) * uint32_t(d.V) + st.v_own, -double(c));
    }
  };

  // ---- superblocks: four blocks whose records (and c) move as one 16-byte access per lane.
  // A lane's 16-byte record load covers the four consecutive samples 4 j .. 4 j + 3 of its tree, so block k of a
  // superblock takes the samples 4 j + k (j = 0 .. SPT - 1) and no record has to change lanes: a wavefront spends 35
  // instead of 44 vector-memory instructions on 256 pairs. Every wavefront takes the same number of superblocks
  // (`rounds`); what is left of the part's samples is worked off block by block below.
  long long s_rest = s_begin;
  {
    const long long stride4 = (long long)kWaves * 4 * SPT;
    const bool aligned = (d.S % 4 == 0) && (s_begin % 4 == 0) && nt == TB &&
                         ((reinterpret_cast<uintptr_t>(rec.a) | reinterpret_cast<uintptr_t>(rec.margin) |
                           reinterpret_cast<uintptr_t>(rec.c)) % 16 == 0);
    const long long rounds = aligned ? (s_end - s_begin) / stride4 : 0;
    if (rounds > 0) {
      typedef uint32_t UInt4 __attribute__((ext_vector_type(4)));
      typedef float Float4 __attribute__((ext_vector_type(4)));
      struct Rec4 {
        UInt4 a;
        Float4 mg;
      };
      struct Loads {
        uint32_t rel[P];
        Float4U gv[P], wv[P];
      };
      const uint32_t goff4 = (uint32_t(4 * jq0) * uint32_t(d.T) + uint32_t(tq)) * M + e0;
      const uint32_t gstep4 = 4u * gstep;
      const long long rec_lane_at = (long long)(t0 + rec_t) * d.S + 4 * rec_j;  // + superblock start
      const long long first4 = s_begin + (long long)wave * 4 * SPT;
      auto load_rec4 = [&](long long r) -> Rec4 {
        const long long at = rec_lane_at + first4 + (r < rounds ? r : rounds - 1) * stride4;  // clamped: re-reads
        Rec4 q;
        q.a = *reinterpret_cast<const UInt4 *>(rec.a + at);
        q.mg = *reinterpret_cast<const Float4 *>(rec.margin + at);
        return q;
      };
      // loads of block k of the superblock at sample sb: gradient rows, then (the keys known) the leaf rows
      auto issue = [&](Loads &ld, long long sb, const Rec4 &q, int k) {
        const float *gbase = gout + ((sb + k) * d.T + t0) * M;
#pragma unroll
        for (int u = 0; u < P; ++u) ld.gv[u] = load_chunk(gbase + u * gstep4 + goff4, false);
        const uint32_t a_k = k == 0 ? q.a[0] : (k == 1 ? q.a[1] : (k == 2 ? q.a[2] : q.a[3]));
        static_for<P>([&](auto u_tag) {
          constexpr int u = decltype(u_tag)::value;
          const uint32_t key = uint32_t(group_bcast<P, u>(int(a_k))) & key_mask;
          const uint32_t r = woff + key * M;
          ld.rel[u] = pack_rel(r, key);
          if (need_c) {
            if constexpr (WLDS) {
              ld.wv[u] = Float4U{w_lds[r], 0.f, 0.f, 0.f};
            } else {
              ld.wv[u] = load_chunk(wbase + r, false);
            }
          }
        });
      };
      // block k consumed: dW terms into LDS, this lane's c of the block returned
      auto consume = [&](Loads &ld, const Rec4 &q, int k) -> float {
        const float mg_k = k == 0 ? q.mg[0] : (k == 1 ? q.mg[1] : (k == 2 ? q.mg[2] : q.mg[3]));
        float c_mine = 0.f;
        static_for<P>([&](auto u_tag) {
          constexpr int u = decltype(u_tag)::value;
          const float mg_u = __int_as_float(group_bcast<P, u>(__float_as_int(mg_k)));
          float g[ROUNDS];
          own_elements(ld.gv[u], g);
          if (dw) {
            const uint32_t row = (Z != 0 ? (ld.rel[u] & 0xFFFFu) : ld.rel[u]) - e0, swz = Z != 0 ? ld.rel[u] >> 16 : 0u;
#pragma unroll
            for (int i = 0; i < ROUNDS; ++i) {
              if (i < Split::BASE || i < my_cnt) {
                const float term = ht_abs(mg_u) * g[i];
                Acc *cell = acc + (row + ((uint32_t(my_begin) + i) ^ swz));
                if (FIXED) term_bound.take(term);
                if (FIXED)
                  atomicAdd(reinterpret_cast<unsigned long long *>(cell), to_fixed(double(term), scale));
                else
                  atomicAdd(reinterpret_cast<double *>(cell), double(term));
              }
            }
          }
          if (need_c) {
            float wl[ROUNDS];
            own_elements(ld.wv[u], wl);
            float partial = 0.f;
#pragma unroll
            for (int i = 0; i < ROUNDS; ++i) {
              const float term = __builtin_fmaf(wl[i], g[i], partial);
              partial = (i < Split::BASE || i < my_cnt) ? term : partial;
            }
            partial = group_sum<float>(partial, P);
            c_mine = (li == u) ? partial : c_mine;
          }
        });
        const float c = ht_sign(mg_k) * c_mine;
        if (need_c && dthr_fold) {
          const uint32_t a_k = k == 0 ? q.a[0] : (k == 1 ? q.a[1] : (k == 2 ? q.a[2] : q.a[3]));
          atomicAdd(acc_thr + uint32_t(rec_t) * uint32_t(d.V) + ((a_k >> rec.vshift) & key_mask), -double(c));
        }
        return c;
      };
      Loads l0, l1;
      Rec4 cur = load_rec4(0), nxt;
      issue(l0, first4, cur, 0);
      for (long long r = 0; r < rounds; ++r) {
        const long long sb = first4 + r * stride4;
        const long long sb_next = first4 + (r + 1 < rounds ? r + 1 : r) * stride4;  // clamped: re-reads
        nxt = load_rec4(r + 1);
        Float4 c4;
        issue(l1, sb, cur, 1);
        c4[0] = consume(l0, cur, 0);
        issue(l0, sb, cur, 2);
        c4[1] = consume(l1, cur, 1);
        issue(l1, sb, cur, 3);
        c4[2] = consume(l0, cur, 2);
        issue(l0, sb_next, nxt, 0);
        c4[3] = consume(l1, cur, 3);
        if (need_c) {
          *reinterpret_cast<Float4 *>(rec.c + rec_lane_at + sb) = c4;
          if (FIXED) {
#pragma unroll
            for (int k = 0; k < 4; ++k) bound_take(c_bound, c4[k]);
          }
        }
        cur = nxt;
      }
      s_rest = s_begin + rounds * stride4;
    }
  }

  // This wavefront's blocks start at first, first + stride, ...; nfull of them are complete (64 existing pairs).
  const long long stride = (long long)kWaves * SPT;
  const long long first = s_rest + (long long)wave * SPT;
  long long nblk = first < s_end ? (s_end - first + stride - 1) / stride : 0;
  long long nfull = 0;
  if (nt == TB && first + SPT <= s_end) nfull = (s_end - SPT - first) / stride + 1;
  if (nt != TB) nfull = 0;

  // ---- complete blocks, software pipelined: while block b is consumed, the gradient rows and weights of block b + 1
  // and the records of block b + 2 are in flight (the kernel is otherwise bound by the latency of two dependent
  // round trips per block: records -> weights).
  if (nfull > 0) {
    bool all_on[P];
#pragma unroll
    for (int u = 0; u < P; ++u) all_on[u] = true;
    auto block_at = [&](long long b) { return first + (b < nfull ? b : nfull - 1) * stride; };  // clamped: re-reads
    Stage s0, s1;
    issue_rec(s0, block_at(0), true);
    issue_g(s0, block_at(0), all_on);
    issue_rec(s1, block_at(1), true);
    issue_w(s0, all_on);
    auto iteration = [&](Stage &cur, Stage &nxt, long long b) {
      issue_rec(cur, block_at(b + 2), true);  // cur's record words were consumed by its issue_w
      issue_g(nxt, block_at(b + 1), all_on);
      issue_w(nxt, all_on);
      compute(cur, block_at(b), true, all_on, std::true_type{});
    };
    long long b = 0;
    for (; b + 1 < nfull; b += 2) {
      iteration(s0, s1, b);
      iteration(s1, s0, b + 1);
    }
    if (b < nfull) iteration(s0, s1, b);
  }
  // ---- the incomplete tail (at most one block per wavefront unless the tree group itself is incomplete)
  for (long long bi = nfull; bi < nblk; ++bi) {
    const long long sblk = first + bi * stride;
    const int ns = int(min<long long>(SPT, s_end - sblk));
    const bool have = rec_t < nt && rec_j < ns;
    bool on[P];
#pragma unroll
    for (int u = 0; u < P; ++u) on[u] = jq0 + u * jstep < ns && tq < nt;
    Stage st;
    issue_rec(st, sblk, have);
    issue_g(st, sblk, on);
    issue_w(st, on);
    compute(st, sblk, have, on, std::false_type{});
  }
  if (FIXED && need_c) publish_c_bound(c_bound, hdr);
  if (FIXED && dw && !second_run) publish_term_bound(term_bound, hdr);
  if (dw || dthr_fold) __syncthreads();
  if (dthr_fold) {
    float *dst = dthr_fold + (long long)t0 * d.V;
    const uint32_t n = uint32_t(nt) * uint32_t(d.V);
    for (uint32_t i = threadIdx.x; i < n; i += kForestThreads) {
      if (dw_atomic) {
        if (acc_thr[i] != 0.0) atomicAdd(dst + i, float(acc_thr[i]));
      } else {
        dst[i] = float(acc_thr[i]);
      }
    }
  }
  if (dw) {
    float *dst = dw + (long long)t0 * LM;
    const uint32_t n = uint32_t(nt) * LM;
    // element i of the table sits in cell at(i) (see the swizzle above)
    auto at = [&](uint32_t i) -> uint32_t {
      if (Z == 0) return i;
      const uint32_t row = i / uint32_t(M), m = i - row * uint32_t(M);
      return i - m + (m ^ swizzle_of(row & uint32_t(d.L - 1)));
    };
    if (FIXED) {
      const unsigned long long *q = reinterpret_cast<const unsigned long long *>(acc);
      if (dw_atomic) {
        for (uint32_t i = threadIdx.x; i < n; i += kForestThreads) {
          const unsigned long long v = q[at(i)];
          if (v != 0ull) atomicAdd(dw_fixed + (long long)t0 * LM + i, v);
        }
      } else {
        for (uint32_t i = threadIdx.x; i < n; i += kForestThreads) dst[i] = from_fixed<float>(q[at(i)], inv_scale);
      }
    } else {
      const double *q = reinterpret_cast<const double *>(acc);
      if (dw_atomic) {
        for (uint32_t i = threadIdx.x; i < n; i += kForestThreads) {
          const double v = q[at(i)];
          if (v != 0.0) atomicAdd(dst + i, float(v));
        }
      } else {
        for (uint32_t i = threadIdx.x; i < n; i += kForestThreads) dst[i] = float(q[at(i)]);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// tree-stationary dW + c for wide leaf rows: float, compact records, M = 4 * P with P a power of two (16 ... 256
// outputs per leaf, e.g. the 8 x 8 tiles of a segmentation head), any K
// ---------------------------------------------------------------------------------------------------------------
// A row of M values is one or more whole 64-byte sectors, so nothing is gained by interleaving trees: a wavefront
// takes 64 / P consecutive samples of ONE tree per step, P adjacent lanes per pair, one 16-byte load of the upstream
// gradient and one of the leaf row per lane, both perfectly coalesced per pair (for K > 1 consecutive samples of a tree
// are even consecutive in memory). Everything that does not depend on the data is a lane constant; the sum over a
// row for c runs over the lanes of a pair with DPP row operations. Two steps are in flight per wavefront.
template <int P>
__device__ __forceinline__ float row_group_sum(float v) {
  if constexpr (P >= 2) v += dpp_swap<0xB1>(v);   // quad_perm [1,0,3,2]
  if constexpr (P >= 4) v += dpp_swap<0x4E>(v);   // quad_perm [2,3,0,1]
  if constexpr (P >= 8) v += dpp_swap<0x141>(v);  // row_half_mirror: the other quad of each 8 lanes
  if constexpr (P >= 16) v += dpp_swap<0x140>(v); // row_mirror: the other half of each 16 lanes
  if constexpr (P >= 32) v += __shfl_xor(v, 16, kWave);
  if constexpr (P >= 64) v += __shfl_xor(v, 32, kWave);
  return v;
}

//
// IMAGE: the upstream gradient is the image [B, T, *size] of which the tile-major [B, T, *tiles, *window] is the
// contraction (tile-shaped outputs per leaf); a lane's four outputs are a 16-byte run of an image row (the window's,
// the padding's and the image's innermost extents are multiples of four), read as zero outside the image.
template <int P, bool FIXED, bool IMAGE>
__global__ __launch_bounds__(kForestThreads) void tree_wide_kernel(ForestDims d, const float *__restrict__ w,
                                                                   const float *__restrict__ gout,
                                                                   Records<float, true> rec, float *dw,
                                                                   unsigned long long *dw_fixed, const DetHeader *hdr,
                                                                   int TB, long long part_size, bool need_c,
                                                                   bool dw_atomic, int num_groups, ImageStore img) {
  typedef typename std::conditional<FIXED, unsigned long long, double>::type Acc;
  constexpr int NP = kWave / P;  // pairs per step
  extern __shared__ __align__(16) unsigned char smem[];
  Acc *acc = reinterpret_cast<Acc *>(smem);
  double scale = 1.0, inv_scale = 1.0;
  if (FIXED) {
    if (hdr->fallback_w) dw = nullptr;
    scale = hdr->scale_w;
    inv_scale = hdr->inv_scale_w;
    if (!dw && !need_c) return;
  }
  const int group = xcd_tree_group(blockIdx.x, num_groups);
  if (group < 0) return;
  const int t0 = group * TB;
  const int nt = min(TB, d.T - t0);
  const uint32_t M = uint32_t(d.M), LM = uint32_t(d.L) * M;
  if (dw) {
    for (uint32_t i = threadIdx.x; i < uint32_t(nt) * LM; i += kForestThreads) acc[i] = Acc(0);
    __syncthreads();
  }
  const long long s_begin = (long long)blockIdx.y * part_size;
  const long long s_end = min(d.S, s_begin + part_size);
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  constexpr int kWaves = kForestThreads / kWave;
  const int pr = lane / P, e0 = (lane & (P - 1)) * 4;  // this lane's pair of a step and its first element of the row
  const uint32_t key_mask = rec.key_mask();

  struct Step {
    long long at;  // record index of this lane's pair
    bool on;
    uint32_t a;
    float mg;
    Float4U gv;
  };
  float c_bound = 0.f;  // FIXED: largest |c| this lane stored
  long long img_sb = -1, img_at = -1, img_base = 0;  // IMAGE: the sample block the cached offsets belong to
  auto issue = [&](Step &st, long long sb, int tl) {
    const long long s_raw = sb + pr;
    st.on = s_raw < s_end;
    const long long s = st.on ? s_raw : s_end - 1;
    st.at = (long long)(t0 + tl) * d.S + s;
    st.a = rec.a[st.at];
    st.mg = rec.margin[st.at];
    if constexpr (IMAGE) {
      // the trees of a group run fastest, so the image offset of this lane's run changes once per nt steps
      if (sb != img_sb) {
        img_sb = sb;
        const long long b = s / d.K;
        img_at = img.offset(int(s - b * d.K), e0);
        img_base = b * d.T * img.plane + img_at;
      }
      const Float4U zero = {0.f, 0.f, 0.f, 0.f};
      st.gv = zero;
      if (img_at >= 0)
        st.gv = __builtin_nontemporal_load(
            reinterpret_cast<const Float4U *>(gout + img_base + (long long)(t0 + tl) * img.plane));
    } else {
      const long long row = d.K == 1 ? (s * d.T + (t0 + tl)) * (long long)M : out_offset(d, s, t0 + tl, 0);
      st.gv = __builtin_nontemporal_load(reinterpret_cast<const Float4U *>(gout + row + e0));
    }
  };
  auto finish = [&](Step &st, int tl) {
    const uint32_t cell = (uint32_t(tl) * uint32_t(d.L) + (st.a & key_mask)) * M + uint32_t(e0);
    if (need_c) {
      const Float4U wv = *reinterpret_cast<const Float4U *>(w + (long long)t0 * LM + cell);
      float partial = wv[0] * st.gv[0];
      partial = __builtin_fmaf(wv[1], st.gv[1], partial);
      partial = __builtin_fmaf(wv[2], st.gv[2], partial);
      partial = __builtin_fmaf(wv[3], st.gv[3], partial);
      const float total = row_group_sum<P>(partial);
      if (st.on && e0 == 0) {
        const float c = ht_sign(st.mg) * total;
        rec.c[st.at] = c;
        if (FIXED) bound_take(c_bound, c);
      }
    }
    if (dw && st.on) {
      const float a = ht_abs(st.mg);
      // In LDS a row is kept transposed, element 4 k + i of the row at slot i * P + k: the P lanes of a pair then hit
      // P consecutive cells in each of the four atomic instructions instead of every fourth cell (half the banks).
      const uint32_t slot = cell - uint32_t(e0) + uint32_t(e0 >> 2);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float term = a * st.gv[i];
        if (FIXED)
          atomicAdd(reinterpret_cast<unsigned long long *>(acc) + slot + i * P, to_fixed(double(term), scale));
        else
          atomicAdd(reinterpret_cast<double *>(acc) + slot + i * P, double(term));
      }
    }
  };

  // steps of this wavefront: (sample block, tree) with the tree running fastest; two in flight
  const long long first = s_begin + (long long)wave * NP;
  const long long stride = (long long)kWaves * NP;
  const long long nblk = first < s_end ? (s_end - first + stride - 1) / stride : 0;
  const long long nsteps = nblk * nt;
  auto where = [&](long long i, long long *sb, int *tl) {
    const long long blk = i / nt;
    *tl = int(i - blk * nt);
    *sb = first + blk * stride;
  };
  Step s0, s1;
  long long sb0 = 0, sb1 = 0;
  int tl0 = 0, tl1 = 0;
  if (nsteps > 0) {
    where(0, &sb0, &tl0);
    issue(s0, sb0, tl0);
  }
  for (long long i = 0; i < nsteps; i += 2) {
    const bool second = i + 1 < nsteps;
    if (second) {
      where(i + 1, &sb1, &tl1);
      issue(s1, sb1, tl1);
    }
    finish(s0, tl0);
    if (i + 2 < nsteps) {
      where(i + 2, &sb0, &tl0);
      issue(s0, sb0, tl0);
    }
    if (second) finish(s1, tl1);
  }
  if (FIXED && need_c) publish_c_bound(c_bound, hdr);

  if (dw) {
    __syncthreads();
    float *dst = dw + (long long)t0 * LM;
    const uint32_t n = uint32_t(nt) * LM;
    // element i of the group's rows sits at its row's transposed slot
    auto at = [&](uint32_t i) { return (i & ~(M - 1u)) + (i & 3u) * uint32_t(P) + ((i & (M - 1u)) >> 2); };
    if (FIXED) {
      const unsigned long long *q = reinterpret_cast<const unsigned long long *>(acc);
      if (dw_atomic) {
        for (uint32_t i = threadIdx.x; i < n; i += kForestThreads)
          if (q[at(i)] != 0ull) atomicAdd(dw_fixed + (long long)t0 * LM + i, q[at(i)]);
      } else {
        for (uint32_t i = threadIdx.x; i < n; i += kForestThreads) dst[i] = from_fixed<float>(q[at(i)], inv_scale);
      }
    } else {
      const double *q = reinterpret_cast<const double *>(acc);
      if (dw_atomic) {
        for (uint32_t i = threadIdx.x; i < n; i += kForestThreads)
          if (q[at(i)] != 0.0) atomicAdd(dst + i, float(q[at(i)]));
      } else {
        for (uint32_t i = threadIdx.x; i < n; i += kForestThreads) dst[i] = float(q[at(i)]);
      }
    }
  }
}

// dThr[t, v] = sum over samples with selected vertex v of -c. One workgroup per tree (x sample parts); where a tree's
// vertex table does not fit LDS (depth 15 and more), `vslices` workgroups per tree, each owning a range of vertices
// and passing over all of the tree's records.
template <typename Real, bool COMPACT, bool FIXED, bool SLICED>
__global__ __launch_bounds__(256) void dthr_kernel(ForestDims d, Records<Real, COMPACT> rec, Real *dthr,
                                                   unsigned long long *dthr_fixed, const DetHeader *hdr,
                                                   long long part_size, bool use_atomic, int vslices) {
  typedef typename std::conditional<FIXED, unsigned long long, double>::type Acc;
  extern __shared__ __align__(16) unsigned char smem[];
  Acc *acc = reinterpret_cast<Acc *>(smem);  // fp64 / int64: fast LDS atomics, and the root vertex is a hot spot
  double scale = 1.0, inv_scale = 1.0;
  if (FIXED) {
    if (hdr->fallback_c) return;
    scale = hdr->scale_c;
    inv_scale = hdr->inv_scale_c;
  }
  const int t = int(blockIdx.x) / vslices, vslice = int(blockIdx.x) - t * vslices;
  const int per_slice = (d.V + vslices - 1) / vslices;
  const uint32_t v_begin = uint32_t(vslice) * uint32_t(per_slice);
  const int nv = max(0, min(per_slice, d.V - int(v_begin)));  // this workgroup's vertices [v_begin, v_begin + nv)
  for (int i = threadIdx.x; i < nv; i += 256) acc[i] = Acc(0);
  __syncthreads();
  const long long s_begin = (long long)blockIdx.y * part_size;
  const long long s_end = min(d.S, s_begin + part_size);
  constexpr int kBatch = 8;  // loads in flight per thread
  // The root and its children are selected far more often than any other vertex; as LDS atomics those hits would
  // serialise on one address, so every lane sums them in registers instead (integer sums in deterministic mode, so
  // the result stays independent of the order).
  constexpr int kTop = 3;
  Acc top[kTop];
#pragma unroll
  for (int k = 0; k < kTop; ++k) top[k] = Acc(0);
  auto add = [&](uint32_t v, Real c) {
    Acc val;
    if constexpr (FIXED)
      val = to_fixed(-double(c), scale);
    else
      val = -double(c);
    if (SLICED && v - v_begin >= uint32_t(nv)) return;  // another slice's vertex
    if (v < uint32_t(kTop)) {
#pragma unroll
      for (int k = 0; k < kTop; ++k) top[k] += v == uint32_t(k) ? val : Acc(0);
    } else {
      atomicAdd(acc + (v - v_begin), val);
    }
  };
  for (long long s0 = s_begin + threadIdx.x; s0 < s_end; s0 += 256 * kBatch) {
    uint32_t v[kBatch];
    Real cv[kBatch];
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
      const long long s = min(s0 + i * 256, s_end - 1);
      const long long at = (long long)t * d.S + s;
      v[i] = rec.vertex(at);
      cv[i] = rec.c[at];
    }
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
      if (s0 + i * 256 >= s_end) break;
      add(v[i], cv[i]);
    }
  }
  // the lanes' sums for the top vertices: reduced over the wavefront, then one atomic each
#pragma unroll
  for (int k = 0; k < kTop; ++k) {
    Acc sum = top[k];
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, kWave);
    if ((threadIdx.x & (kWave - 1)) == 0 && vslice == 0 && k < nv) atomicAdd(acc + k, sum);
  }
  __syncthreads();
  Real *dst = dthr + (long long)t * d.V + v_begin;
  for (int i = threadIdx.x; i < nv; i += 256) {
    if (FIXED) {
      const unsigned long long q = reinterpret_cast<const unsigned long long *>(acc)[i];
      if (use_atomic) {
        if (q != 0ull) atomicAdd(dthr_fixed + (long long)t * d.V + v_begin + i, q);
      } else {
        dst[i] = from_fixed<Real>(q, inv_scale);
      }
    } else {
      const double q = reinterpret_cast<const double *>(acc)[i];
      if (use_atomic) {
        if (q != 0.0) atomicAdd(dst + i, Real(q));
      } else {
        dst[i] = Real(q);
      }
    }
  }
}

// dX: sample tile x all trees. LDS accumulator [F][BT+1] (the pad keeps the transposing write-out conflict free).
// FIXED: 64-bit fixed-point cells; dX is cleared beforehand and left alone when the header asks for the fallback.
// A feature space too wide for the tile is served in windows of f_per features (blockIdx.y): every window passes
// over all records of the tile's samples and keeps the terms whose ordinal falls inside it.
template <typename Real, int BT, bool COMPACT, bool FIXED, bool WINDOWED>
__global__ __launch_bounds__(kForestThreads) void dx_kernel(ForestDims d, Records<Real, COMPACT> rec, Real *dx,
                                                            const DetHeader *hdr, int f_per) {
  typedef typename std::conditional<FIXED, unsigned long long, Real>::type Acc;
  constexpr int NT = kForestThreads;
  constexpr int TC = NT / BT;
  constexpr int LD = BT + 1;
  extern __shared__ __align__(16) unsigned char smem[];
  Acc *acc = reinterpret_cast<Acc *>(smem);
  double scale = 1.0, inv_scale = 1.0;
  if (FIXED) {
    if (hdr->fallback_c) return;
    scale = hdr->scale_c;
    inv_scale = hdr->inv_scale_c;
  }
  const uint32_t f_begin = WINDOWED ? blockIdx.y * uint32_t(f_per) : 0u;
  const uint32_t nf = WINDOWED ? uint32_t(min(f_per, d.F - int(f_begin))) : uint32_t(d.F);  // features [f_begin, f_begin + nf)
  for (int i = threadIdx.x; i < int(nf) * LD; i += NT) acc[i] = Acc(0);
  __syncthreads();
  const long long s0 = (long long)blockIdx.x * BT;
  const int j = threadIdx.x % BT, tt = threadIdx.x / BT;
  const long long s = s0 + j;
  // Packed records of a sample count that is a multiple of four: a lane takes four consecutive samples of a tree with
  // one 16-byte load of the record words and one of c, a quarter of the vector-memory instructions of the
  // sample-per-lane loop below (which costs the CU ~16 cycles per instruction however few bytes it moves).
  bool quads = false;
  if constexpr (COMPACT && BT % 4 == 0) {
    quads = rec.oshift != 0 && d.S % 4 == 0 && reinterpret_cast<uintptr_t>(rec.a) % 16 == 0 &&
            reinterpret_cast<uintptr_t>(rec.c) % (4 * sizeof(Real)) == 0;
  }
  if constexpr (COMPACT && BT % 4 == 0) {
    if (quads) {
      typedef uint32_t Word4 __attribute__((ext_vector_type(4)));
      typedef Real Real4 __attribute__((ext_vector_type(4)));
      constexpr int LPT = BT / 4;    // lanes per tree
      constexpr int TCQ = NT / LPT;  // trees in flight per pass of the workgroup
      constexpr int kBatchQ = 4;
      const int jq = 4 * (threadIdx.x % LPT), tq = threadIdx.x / LPT;
      if (s0 + jq < d.S) {
        for (int t0 = tq; t0 < d.T; t0 += TCQ * kBatchQ) {
          Word4 av[kBatchQ];
          Real4 cv[kBatchQ];
#pragma unroll
          for (int i = 0; i < kBatchQ; ++i) {
            const int t = min(t0 + i * TCQ, d.T - 1);
            const long long at = (long long)t * d.S + s0 + jq;
            av[i] = *reinterpret_cast<const Word4 *>(rec.a + at);
            cv[i] = __builtin_nontemporal_load(reinterpret_cast<const Real4 *>(rec.c + at));
          }
#pragma unroll
          for (int i = 0; i < kBatchQ; ++i) {
            if (t0 + i * TCQ >= d.T) break;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const uint32_t o = (av[i][e] >> rec.oshift) - f_begin;
              if (WINDOWED && o >= nf) continue;
              if (FIXED)
                atomicAdd(reinterpret_cast<unsigned long long *>(acc) + o * LD + jq + e,
                          to_fixed(double(cv[i][e]), scale));
              else
                lds_add(reinterpret_cast<Real *>(acc) + o * LD + jq + e, cv[i][e]);
            }
          }
        }
      }
    }
  }
  if (!quads && s < d.S) {
    // the loads of several trees are issued together: the loop is otherwise bound by one memory round trip per tree
    constexpr int kBatch = 8;
    for (int t0 = tt; t0 < d.T; t0 += TC * kBatch) {
      uint32_t o[kBatch];
      Real cv[kBatch];
#pragma unroll
      for (int i = 0; i < kBatch; ++i) {
        const int t = min(t0 + i * TC, d.T - 1);
        const long long at = (long long)t * d.S + s;
        o[i] = rec.ord(at) - f_begin;
        cv[i] = __builtin_nontemporal_load(rec.c + at);
      }
#pragma unroll
      for (int i = 0; i < kBatch; ++i) {
        if (t0 + i * TC >= d.T) break;
        if (WINDOWED && o[i] >= nf) continue;
        if (FIXED)
          atomicAdd(reinterpret_cast<unsigned long long *>(acc) + o[i] * LD + j, to_fixed(double(cv[i]), scale));
        else
          lds_add(reinterpret_cast<Real *>(acc) + o[i] * LD + j, cv[i]);
      }
    }
  }
  __syncthreads();
  auto cell = [&](int f, int jj) -> Real {
    if (FIXED) return from_fixed<Real>(reinterpret_cast<const unsigned long long *>(acc)[f * LD + jj], inv_scale);
    return reinterpret_cast<const Real *>(acc)[f * LD + jj];
  };
  if (d.K == 1) {
    // dx[s, 0..F) is a contiguous row: a wavefront per sample, lanes along the features
    const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
    for (int jj = wv; jj < BT && s0 + jj < d.S; jj += NT / kWave) {
      Real *row = dx + (s0 + jj) * d.F + f_begin;
      for (int f = lane; f < int(nf); f += kWave) row[f] = cell(f, jj);
    }
  } else {
    // dx[b, f, k]: consecutive samples of a tile are consecutive k (within one b)
    for (int i = threadIdx.x; i < int(nf) * BT; i += NT) {
      const int f = i / BT, jj = i - f * BT;
      const long long ss = s0 + jj;
      if (ss < d.S) dx[(ss / d.K) * d.FK + (long long)(f_begin + f) * d.K + (ss % d.K)] = cell(f, jj);
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// fused kernel with global atomics (small problems, depth > 16, F > 65536, huge leaf tables)
// ---------------------------------------------------------------------------------------------------------------
template <typename Real, bool FERN, int BT, bool XLDS>
__global__ __launch_bounds__(kForestThreads) void backward_fused_kernel(
    ForestDims d, const Real *__restrict__ x, const Node<Real> *__restrict__ nodes, const Real *__restrict__ w,
    const Real *__restrict__ gout, Real *__restrict__ dx, Real *__restrict__ dthr, Real *__restrict__ dw,
    int trees_per_block, FastDiv div_m) {
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
      const Node<Real> *nd[1] = {nodes + (long long)t * d.V};
      WalkResult<Real> r[1];
      if (XLDS)
        walk_many<Real, FERN, 1>(d.depth, nd, [&](int, int f) { return xs[f * BT + j]; }, r);
      else
        walk_many<Real, FERN, 1>(d.depth, nd, [&](int, int f) { return x[xbase + (long long)f * d.K]; }, r);
      r_margin[tt * BT + j] = r[0].margin;
      r_key[tt * BT + j] = r[0].key;
      r_vertex[tt * BT + j] = r[0].vertex;
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
        const int lo = div_m.div(r), m = r - lo * d.M;
        const int jj = k1 ? hi : lo, t2 = k1 ? lo : hi;
        const long long ss = s0 + jj;
        if (ss < d.S) {
          const Real g = gout[out_offset(d, ss, tb + t2, m)];
          const uint32_t key = r_key[t2 * BT + jj];
          const long long wi = ((long long)(tb + t2) * d.L + key) * d.M + m;
          if (dw) atomicAdd(dw + wi, ht_abs(r_margin[t2 * BT + jj]) * g);
          if (need_c) lds_add(r_csum + t2 * BT + jj, w[wi] * g);
        }
      }
    }
    __syncthreads();

    if (mine && need_c) {
      const Real c = ht_sign(r_margin[tt * BT + j]) * r_csum[tt * BT + j];
      const uint32_t v = r_vertex[tt * BT + j];
      const long long o = nodes[(long long)t * d.V + v].ord;
      if (dx) atomicAdd(dx + xbase + o * d.K, c);
      if (dthr) atomicAdd(dthr + (long long)t * d.V + v, -c);
    }
    __syncthreads();
  }
}

template <typename Real, bool FERN, int BT, bool XLDS>
int launch_backward_fused(const ForestDims &d, const Real *x, const Node<Real> *nodes, const Real *w, const Real *gout,
                          Real *dx, Real *dthr, Real *dw, hipStream_t stream) {
  constexpr int TC = kForestThreads / BT;
  const size_t lds =
      (XLDS ? size_t(d.F) * BT * sizeof(Real) : 0) + size_t(TC) * BT * (2 * sizeof(Real) + 2 * sizeof(uint32_t));
  const long long tiles = (d.S + BT - 1) / BT;
  int trees_per_block, gy;
  split_trees(tiles, d.T, TC, &trees_per_block, &gy);
  if (tiles > 0x7fffffffLL) return fail(HT_ERR_RUNTIME, "Error: too many sample tiles for one launch.");
  auto kernel = backward_fused_kernel<Real, FERN, BT, XLDS>;
  HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));
  hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)gy), dim3(kForestThreads), lds, stream, d, x, nodes, w, gout,
                     dx, dthr, dw, trees_per_block, FastDiv(d.M));
  HT_LAUNCH_CHECK("forest backward (fused, atomics)");
  return HT_OK;
}

template <typename Real, bool FERN>
int dispatch_backward_fused(const ForestDims &d, const Real *x, const Node<Real> *nodes, const Real *w,
                            const Real *gout, Real *dx, Real *dthr, Real *dw, hipStream_t stream) {
  const size_t reserve = 32 * 1024;
  switch (pick_tile<Real>(d.F, reserve)) {
    case 64: return launch_backward_fused<Real, FERN, 64, true>(d, x, nodes, w, gout, dx, dthr, dw, stream);
    case 32: return launch_backward_fused<Real, FERN, 32, true>(d, x, nodes, w, gout, dx, dthr, dw, stream);
    case 16: return launch_backward_fused<Real, FERN, 16, true>(d, x, nodes, w, gout, dx, dthr, dw, stream);
    case 8: return launch_backward_fused<Real, FERN, 8, true>(d, x, nodes, w, gout, dx, dthr, dw, stream);
    default: return launch_backward_fused<Real, FERN, 64, false>(d, x, nodes, w, gout, dx, dthr, dw, stream);
  }
}

// ---------------------------------------------------------------------------------------------------------------
// deterministic owner-computes kernels (consume the records)
// ---------------------------------------------------------------------------------------------------------------
// dX: thread per sample, trees in index order, one add per (tree, m) term straight into the owned cell: the same
// sequence of roundings as the reference CPU loop (hingetree.cpp:236-254).
template <typename Real, bool COMPACT>
__global__ __launch_bounds__(256) void det_dx_kernel(ForestDims d, const Real *__restrict__ w,
                                                     const Real *__restrict__ gout, Records<Real, COMPACT> rec,
                                                     Real *dx, const int *run_if) {
  if (run_if && *run_if == 0) return;
  const long long s = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (s >= d.S) return;
  const long long b = s / d.K, k = s % d.K;
  const long long xbase = b * d.FK + k;
  for (int t = 0; t < d.T; ++t) {
    const long long at = (long long)t * d.S + s;
    const uint32_t key = rec.key(at);
    const Real sg = ht_sign(rec.margin[at]);
    const long long o = rec.ord(at);
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
template <typename Real, bool LDS_ACC, bool COMPACT>
__global__ __launch_bounds__(kWave) void det_tree_kernel(ForestDims d, const Real *__restrict__ w,
                                                         const Real *__restrict__ gout, Records<Real, COMPACT> rec,
                                                         Real *dthr, Real *dw, const int *run_if) {
  extern __shared__ __align__(16) unsigned char smem[];
  if (run_if && *run_if == 0) return;
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
      key = rec.key(at);
      v = rec.vertex(at);
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

// ---------------------------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------------------------
constexpr int kLeanMaxOutputs = 16;  // tree_lean_kernel: at most four lanes of four values per pair
// Elements of a leaf row that a wavefront's 64 lanes cover with one 16-byte chunk each: wider rows take the tree kernel
// several launches, one per window of this many elements (at most kMaxRowWindows of them).
template <typename Real>
constexpr int row_window() {
  return kWave * (16 / int(sizeof(Real)));
}
constexpr int kMaxRowWindows = 4;
struct TreePlan {
  int TB;               // trees per workgroup
  int groups, parts;    // grid (groups counts tree groups x leaf slices)
  long long part_size;  // samples per part
  size_t lds;
  int slices;           // > 1: a tree's leaf table is split over that many workgroups (generic tree kernel only)
};
constexpr int kMaxLeafSlices = 1024;

// Single-output leaf tables (M == 1, 4 bytes per leaf) are small enough to sit in LDS next to the accumulators of the
// lean tree kernel; its leaf-weight gathers then never leave the CU.
static inline size_t staged_weights_per_tree(const ForestDims &d, bool lean) {
  return lean && d.M == 1 ? size_t(d.L) * sizeof(float) : 0;
}

// row_limit: the elements of a leaf row that one launch of the tree kernel accumulates (row_window below).
static bool plan_trees(const ForestDims &d, bool need_dw, bool lean, TreePlan *p, int row_limit) {
  const size_t per_tree = size_t(d.L) * (d.M < row_limit ? d.M : row_limit) * sizeof(double);
  const size_t w_tree = staged_weights_per_tree(d, lean);
  int tb = 4;
  p->slices = 1;
  if (need_dw) {
    if (per_tree > size_t(kLdsBytes)) {
      // one tree's table is too large: slices of its leaves (a power of two of them, like the leaves), one tree at a time
      int slices = 2;
      while (per_tree / slices > size_t(kLdsBytes) && slices < d.L) slices *= 2;
      if (per_tree / slices > size_t(kLdsBytes) || slices > kMaxLeafSlices || slices > d.L) return false;
      p->slices = slices;
      p->TB = 1;
      p->groups = d.T * slices;
      p->parts = 1;
      p->part_size = d.S;
      if (p->groups < kNumCUs) {
        long long parts = (kNumCUs + p->groups - 1) / p->groups;
        const long long max_parts = (d.S + 4 * kForestThreads - 1) / (4 * kForestThreads);
        if (parts > max_parts) parts = max_parts;
        if (parts < 1) parts = 1;
        p->part_size = (d.S + parts - 1) / parts;
        p->parts = int((d.S + p->part_size - 1) / p->part_size);
      }
      p->lds = per_tree / slices;
      return true;
    }
    tb = int(size_t(kLdsBytes) / per_tree);
  }
  if (w_tree != 0) {
    // room for the staged weights and the vertex table of the group as well
    const size_t all = (need_dw ? per_tree : 0) + w_tree + size_t(d.V) * sizeof(double);
    int fit = int(size_t(kLdsBytes - 64) / all);
    if (fit < 1) fit = 1;
    if (tb > fit) tb = fit;
  }
  if (tb > kMaxGroupTrees) tb = kMaxGroupTrees;
  if (tb > d.T) tb = d.T;
  // the lean kernel (see lean_tree_ok) wants a power of two
  const bool pow2 = lean && d.M <= kLeanMaxOutputs;
  if (pow2)
    while (tb & (tb - 1)) tb &= tb - 1;
  // Keep at least ~one workgroup per CU by shrinking the groups before splitting the samples -- except for leaves
  // with few outputs, where a group reads only 4 * M * TB bytes of every 128-byte line of upstream gradients it
  // requests: there wide groups matter more, and the samples are split instead.
  const bool keep = w_tree != 0 || (pow2 && d.M <= 4);
  while (!keep && tb > 4 && (d.T + tb - 1) / tb < kNumCUs) tb = (tb + 1) / 2;
  p->TB = tb;
  p->groups = (d.T + tb - 1) / tb;
  long long parts = 1;
  if (p->groups < kNumCUs) parts = (kNumCUs + p->groups - 1) / p->groups;
  const long long max_parts = (d.S + 4 * kForestThreads - 1) / (4 * kForestThreads);  // >= 4 samples per thread
  if (p->groups < kNumCUs) {
    // The split that leaves the fewest CUs idle in the last round. An XCD (32 CUs) takes ceil(groups / 8) of the tree
    // groups, each times the sample parts, and a CU holds as many of these workgroups as its LDS and its 2048 thread
    // slots allow.
    const size_t lds = size_t(tb) * ((need_dw ? per_tree : 0) + (keep ? w_tree + size_t(d.V) * sizeof(double) : 0));
    const long long per_cu = lds * 2 <= size_t(kLdsBytes) ? 2 : 1;
    const long long cap = per_cu * (kNumCUs / kNumXCDs);
    const long long xcd_groups = (p->groups + kNumXCDs - 1) / kNumXCDs;
    double best = -1.0;
    for (long long c = 1; c <= 16 && c <= max_parts; ++c) {
      const long long rounds = (xcd_groups * c + cap - 1) / cap;
      const double eff = double(c * p->groups) / double(rounds * cap * kNumXCDs);
      if (eff > best + 0.02) best = eff, parts = c;
    }
  }
  if (parts > max_parts) parts = max_parts;
  if (parts < 1) parts = 1;
  if (parts > 65535) parts = 65535;
  p->part_size = (d.S + parts - 1) / parts;
  p->parts = int((d.S + p->part_size - 1) / p->part_size);
  p->lds = need_dw ? size_t(tb) * per_tree : 0;
  return true;
}

// Sample parts of the dThr kernel: one workgroup per tree unless the trees alone cannot fill the device.
static void plan_dthr(const ForestDims &d, long long *part_size, int *gy) {
  long long parts = d.T >= 2 * kNumCUs ? 1 : (2 * kNumCUs + d.T - 1) / d.T;
  const long long max_parts = (d.S + 1023) / 1024;
  if (parts > max_parts) parts = max_parts;
  if (parts < 1) parts = 1;
  if (parts > 65535) parts = 65535;
  *part_size = (d.S + parts - 1) / parts;
  *gy = int((d.S + *part_size - 1) / *part_size);
}

template <typename Real, bool COMPACT, bool FIXED, int U>
int launch_tree_kernel_u(const ForestDims &d, const TreePlan &p, int P, const Real *w, const Real *gout,
                         Records<Real, COMPACT> rec, Real *dw, unsigned long long *dw_fixed, const DetHeader *hdr,
                         bool need_c, hipStream_t stream, int m0, int Mw) {
  auto kernel = tree_kernel<Real, COMPACT, FIXED, U>;
  HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));
  const int per_xcd = (p.groups + kNumXCDs - 1) / kNumXCDs;
  hipLaunchKernelGGL(kernel, dim3((unsigned)(per_xcd * kNumXCDs), (unsigned)p.parts), dim3(kForestThreads), p.lds,
                     stream, d, w, gout, rec, dw, dw_fixed, hdr, p.TB, p.part_size, need_c, p.parts > 1, P, p.groups,
                     p.slices, m0, Mw);
  HT_LAUNCH_CHECK("forest backward (trees)");
  return HT_OK;
}

// Shapes of tree_wide_kernel: M = 4 * P with P a power of two from 4 to 64, leaf offsets of a tree group in 32 bits.
static bool wide_rows_ok(const ForestDims &d, const TreePlan &p) {
  const int P4 = d.M / 4;
  return p.slices == 1 && d.M % 4 == 0 && P4 >= 4 && P4 <= kWave && (P4 & (P4 - 1)) == 0 &&
         (long long)p.TB * d.L * d.M < (1ll << 31);
}

// Shapes of tree_lean_kernel (float, compact records): contiguous rows of up to 16 outputs, a power-of-two tree group,
// 32-bit offsets inside a block and a group.
static bool lean_tree_ok(const ForestDims &d, const TreePlan &p, int *log2_tb_out) {
  int log2_tb = 0;
  while ((1 << (log2_tb + 1)) <= p.TB) ++log2_tb;
  if (log2_tb_out) *log2_tb_out = log2_tb;
  return p.slices == 1 && d.K == 1 && (1 << log2_tb) == p.TB && p.TB <= 16 && (long long)kWave * d.T * d.M < (1ll << 31) &&
         (long long)p.TB * d.L * d.M < (1ll << 31) && d.M >= 1 && d.M <= kLeanMaxOutputs;
}

// gout_image: the upstream gradient is stored as the image of the tile geometry (only tree_wide_kernel reads it so).
// second_run: the repeat of the lean kernel after a sampled bound was exceeded (see DetHeader); it does nothing
// unless the header asks for it.
template <typename Real, bool COMPACT, bool FIXED>
int launch_tree_kernel(const ForestDims &d, const TreePlan &p, const Real *w, const Real *gout,
                       Records<Real, COMPACT> rec, Real *dw, unsigned long long *dw_fixed, const DetHeader *hdr,
                       bool need_c, Real *dthr, bool *dthr_done, hipStream_t stream, const ImageStore *gout_image,
                       bool second_run = false) {
  *dthr_done = false;
  if constexpr (std::is_same<Real, float>::value && COMPACT) {
    if (gout_image != nullptr &&
        (d.K == 1 || !wide_rows_ok(d, p) || reinterpret_cast<uintptr_t>(gout) % 16 != 0 ||
         reinterpret_cast<uintptr_t>(w) % 16 != 0))
      return fail(HT_ERR_RUNTIME, "Error: this shape cannot read the upstream gradient as an image.");
  } else {
    if (gout_image != nullptr)
      return fail(HT_ERR_RUNTIME, "Error: this shape cannot read the upstream gradient as an image.");
  }
  if constexpr (std::is_same<Real, float>::value && COMPACT) {
    int log2_tb = 0;
    if (lean_tree_ok(d, p, &log2_tb)) {
      // dThr rides along where its fp64 table fits behind the leaf accumulators (atomic mode: the fixed-point scale of
      // c is only known once every c exists)
      const size_t acc_lds = dw ? size_t(p.TB) * d.L * d.M * sizeof(double) : 0;
      const size_t thr_off = align_up(acc_lds, 16), thr_lds = size_t(p.TB) * d.V * sizeof(double);
      const size_t w_lds = size_t(p.TB) * staged_weights_per_tree(d, true);
      const bool stage_w = w_lds != 0 && need_c && thr_off + thr_lds + w_lds <= size_t(kLdsBytes);
      const bool fold = !FIXED && dthr != nullptr && need_c &&
                        thr_off + thr_lds + (stage_w ? w_lds : 0) <= size_t(kLdsBytes);
      const size_t w_off = fold ? thr_off + thr_lds : thr_off;
      size_t lds = stage_w ? w_off + w_lds : (fold ? thr_off + thr_lds : acc_lds);
      if (lds < p.lds) lds = p.lds;
      float *dthr_fold = fold ? dthr : nullptr;
      *dthr_done = fold;
      const int per_xcd = (p.groups + kNumXCDs - 1) / kNumXCDs;
      const dim3 grid((unsigned)(per_xcd * kNumXCDs), (unsigned)p.parts);
#define HT_LEAN_LAUNCH(MM, WLDS_)                                                                                     \
  {                                                                                                                   \
    auto kernel = tree_lean_kernel<MM, FIXED, WLDS_>;                                                                 \
    HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));                          \
    hipLaunchKernelGGL(kernel, grid, dim3(kForestThreads), lds, stream, d, w, gout, rec, dw, dw_fixed, hdr, log2_tb,  \
                       p.part_size, need_c, p.parts > 1, p.groups, dthr_fold, uint32_t(thr_off), uint32_t(w_off),     \
                       second_run);                                                                                   \
  }
#define HT_LEAN(MM) \
  case MM: HT_LEAN_LAUNCH(MM, false) break;
      switch (d.M) {
        case 1:
          if (stage_w) HT_LEAN_LAUNCH(1, true) else HT_LEAN_LAUNCH(1, false)
          break;
        HT_LEAN(2) HT_LEAN(3) HT_LEAN(4) HT_LEAN(5) HT_LEAN(6) HT_LEAN(7) HT_LEAN(8) HT_LEAN(9) HT_LEAN(10)
        HT_LEAN(11) HT_LEAN(12) HT_LEAN(13) HT_LEAN(14) HT_LEAN(15) HT_LEAN(16)
      }
#undef HT_LEAN
#undef HT_LEAN_LAUNCH
      HT_LAUNCH_CHECK("forest backward (trees)");
      return HT_OK;
    }
  }
  if constexpr (std::is_same<Real, float>::value && COMPACT) {
    // wide leaf rows: M = 4 * P, P a power of two
    const int P4 = d.M / 4;
    if (wide_rows_ok(d, p) && reinterpret_cast<uintptr_t>(gout) % 16 == 0 &&
        reinterpret_cast<uintptr_t>(w) % 16 == 0) {
      const ImageStore img = gout_image ? *gout_image : ImageStore{};
      const int per_xcd = (p.groups + kNumXCDs - 1) / kNumXCDs;
      const dim3 grid((unsigned)(per_xcd * kNumXCDs), (unsigned)p.parts);
#define HT_WIDE(PP)                                                                                                   \
  case PP: {                                                                                                          \
    auto kernel = gout_image ? tree_wide_kernel<PP, FIXED, true> : tree_wide_kernel<PP, FIXED, false>;                \
    HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));                        \
    hipLaunchKernelGGL(kernel, grid, dim3(kForestThreads), p.lds, stream, d, w, gout, rec, dw, dw_fixed, hdr, p.TB,   \
                       p.part_size, need_c, p.parts > 1, p.groups, img);                                              \
    break;                                                                                                            \
  }
      switch (P4) {
        HT_WIDE(4)
        HT_WIDE(8)
        HT_WIDE(16)
        HT_WIDE(32)
        HT_WIDE(64)
      }
#undef HT_WIDE
      HT_LAUNCH_CHECK("forest backward (trees, wide rows)");
      return HT_OK;
    }
  }
  constexpr int VE = 16 / sizeof(Real);
  // one launch per window of the leaf rows (a single one unless a row is wider than a wavefront's 64 chunks)
  for (int m0 = 0; m0 < d.M; m0 += row_window<Real>()) {
    const int Mw = d.M - m0 < row_window<Real>() ? d.M - m0 : row_window<Real>();
    const int Q = Mw >= VE ? (Mw + VE - 1) / VE : 1;  // 16-byte chunks in one pair's values
    int P = 1;                                        // lanes per pair
    while (P < Q) P <<= 1;
    int rc;
    if (P >= 4)
      rc = launch_tree_kernel_u<Real, COMPACT, FIXED, 4>(d, p, P, w, gout, rec, dw, dw_fixed, hdr, need_c, stream, m0, Mw);
    else if (P == 2)
      rc = launch_tree_kernel_u<Real, COMPACT, FIXED, 2>(d, p, P, w, gout, rec, dw, dw_fixed, hdr, need_c, stream, m0, Mw);
    else
      rc = launch_tree_kernel_u<Real, COMPACT, FIXED, 1>(d, p, P, w, gout, rec, dw, dw_fixed, hdr, need_c, stream, m0, Mw);
    if (rc != HT_OK) return rc;
  }
  return HT_OK;
}

template <typename Real, int BT, bool COMPACT, bool FIXED>
int launch_dx(const ForestDims &d, Records<Real, COMPACT> rec, Real *dx, const DetHeader *hdr, hipStream_t stream) {
  const size_t cell = (BT + 1) * (FIXED ? sizeof(unsigned long long) : sizeof(Real));  // bytes per feature
  int f_per = d.F;  // features per workgroup: all of them, or as many as LDS holds
  if (size_t(f_per) * cell > size_t(kLdsBytes)) f_per = int(size_t(kLdsBytes) / cell);
  const int windows = (d.F + f_per - 1) / f_per;
  const size_t lds = size_t(f_per) * cell;
  const long long tiles = (d.S + BT - 1) / BT;
  if (tiles > 0x7fffffffLL || windows > 65535) return fail(HT_ERR_RUNTIME, "Error: too many sample tiles for one launch.");
  auto kernel = dx_kernel<Real, BT, COMPACT, FIXED, false>;
  if constexpr (BT == 8) {  // (windows are only ever needed on the smallest tile)
    if (windows > 1) kernel = dx_kernel<Real, BT, COMPACT, FIXED, true>;
  }
  if (BT != 8 && windows > 1) return fail(HT_ERR_RUNTIME, "Error: feature windows on a tile other than the smallest.");
  HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));
  hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)windows), dim3(kForestThreads), lds, stream, d, rec, dx, hdr,
                     f_per);
  HT_LAUNCH_CHECK("forest backward (dX)");
  return HT_OK;
}

// Largest dX tile whose padded [F][BT+1] accumulator of `cell`-byte cells fits LDS; 0 if none.
static int pick_dx_tile(int F, size_t cell) {
  const int candidates[4] = {64, 32, 16, 8};
  for (int bt : candidates)
    if (size_t(F) * (bt + 1) * cell <= size_t(kLdsBytes)) return bt;
  return 0;
}

template <typename Real>
bool staged_ok(const ForestDims &d, bool need_dx, bool need_dw, bool fixed) {
  if (d.M < 1) return false;
  // a leaf row is served in at most kMaxRowWindows windows of a wavefront's 64 chunks of 16 bytes, and the tree kernel
  // addresses the gradient rows of one 64-sample step with 32-bit offsets
  if (d.M > kMaxRowWindows * row_window<Real>()) return false;
  if ((long long)d.T * d.M * kWave >= (1ll << 31)) return false;
  // (a leaf table beyond LDS is accumulated in slices of its leaves, each at least one leaf row)
  if (need_dw && size_t(d.L) * d.M * sizeof(double) > size_t(kLdsBytes) * kMaxLeafSlices) return false;
  if (need_dw && size_t(d.M) * sizeof(double) > size_t(kLdsBytes)) return false;
  if ((long long)d.L * d.M >= (1ll << 31)) return false;
  // (a vertex table beyond LDS is accumulated in slices of its vertices)
  if (size_t(d.V) * sizeof(double) > size_t(kLdsBytes) * 64) return false;
  // (dX of a feature space too wide for the tile: windows of features, at most 65535 of them)
  if (need_dx && (long long)d.F * 9 * 8 > (long long)kLdsBytes * 65535) return false;
  return true;
}

// Problems this small finish sooner in the single fused kernel than in four launches.
static bool prefer_fused(const ForestDims &d) { return double(d.S) * double(d.T) < double(1 << 18); }

// Extra workspace of the fixed-point deterministic pass behind the records: header, then the integer dW and dThr
// buffers that merge sample parts (present only when the respective kernel splits the samples).
struct FixedLayout {
  size_t header, dw, dthr, total;
};
static FixedLayout fixed_layout(const ForestDims &d, bool need_dthr, bool need_dw, bool lean, int row_limit) {
  FixedLayout l{};
  TreePlan plan;
  l.header = 0;
  size_t at = kDetHeaderBytes;
  l.dw = at;
  if (need_dw && plan_trees(d, true, lean, &plan, row_limit) && plan.parts > 1) at += align_up(size_t(d.T) * d.L * d.M * 8, 256);
  l.dthr = at;
  long long part_size;
  int gy;
  plan_dthr(d, &part_size, &gy);
  if (need_dthr && gy > 1) at += align_up(size_t(d.T) * d.V * 8, 256);
  l.total = at;
  return l;
}

template <typename Real>
int launch_absmax(const Real *p, long long n, unsigned long long *slot, hipStream_t stream) {
  if (n <= 0) return HT_OK;
  long long blocks = (n / (16 / (long long)sizeof(Real)) + kAbsmaxThreads - 1) / kAbsmaxThreads;
  if (blocks > 8 * kNumCUs) blocks = 8 * kNumCUs;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL((absmax_kernel<Real>), dim3((unsigned)blocks), dim3(kAbsmaxThreads), 0, stream, p, n, slot);
  HT_LAUNCH_CHECK("forest backward (magnitude bound)");
  return HT_OK;
}

// Staged pipeline over the records `rec`, which are produced here first (walk) or came from a forward pass. FIXED selects the bit-reproducible fixed-point accumulators; fixed_ws then points at the
// FixedLayout area and dX must have been cleared by the caller.
template <typename Real, bool FERN, bool COMPACT, bool FIXED>
int backward_staged(const ForestDims &d, const Real *x, const Node<Real> *nodes, const Real *w, const Real *gout,
                    Real *dx, Real *dthr, Real *dw, Records<Real, COMPACT> rec, bool walk, void *fixed_ws,
                    hipStream_t stream, const ImageStore *gout_image = nullptr, bool keep_c = false) {
  int rc = HT_OK;
  if (FIXED && gout_image != nullptr)
    return fail(HT_ERR_RUNTIME, "Error: the deterministic mode cannot read the upstream gradient as an image.");
  if (walk && (rc = dispatch_records<Real, FERN, COMPACT>(d, x, nodes, rec, stream)) != HT_OK) return rc;
  const bool need_c = dx || dthr || keep_c;  // keep_c: the caller goes on from c itself
  const long long pairs = (long long)d.T * d.S;
  TreePlan plan;
  constexpr bool kLean = std::is_same<Real, float>::value && COMPACT;
  if (!plan_trees(d, dw != nullptr, kLean && d.K == 1, &plan, row_window<Real>()))
    return fail(HT_ERR_RUNTIME, "Error: leaf table too large.");
  long long dthr_part;
  int dthr_gy;
  plan_dthr(d, &dthr_part, &dthr_gy);

  DetHeader *hdr = nullptr;
  unsigned long long *dw_fixed = nullptr, *dthr_fixed = nullptr;
  bool sampled = false;  // the scale of dW rests on a sample of the upstream gradient (see DetHeader)
  if (FIXED) {
    const FixedLayout lay = fixed_layout(d, dthr != nullptr, dw != nullptr, kLean && d.K == 1, row_window<Real>());
    unsigned char *base = static_cast<unsigned char *>(fixed_ws);
    hdr = reinterpret_cast<DetHeader *>(base + lay.header);
    dw_fixed = reinterpret_cast<unsigned long long *>(base + lay.dw);
    dthr_fixed = reinterpret_cast<unsigned long long *>(base + lay.dthr);
    hipLaunchKernelGGL(det_init_kernel, dim3(1), dim3(256), 0, stream, hdr);
    HT_LAUNCH_CHECK("forest backward (deterministic header)");
    if (dw) {
      sampled = kLean && lean_tree_ok(d, plan, nullptr) && reinterpret_cast<uintptr_t>(gout) % 16 == 0 &&
                size_t(pairs) * d.M * sizeof(Real) >= kSampleMinBytes;
      if (sampled) {
        const long long runs = pairs * d.M / (16 / (long long)sizeof(Real)) / kWave / kSampleEvery;
        long long blocks = (runs + kAbsmaxThreads / kWave - 1) / (kAbsmaxThreads / kWave);
        if (blocks > 8 * kNumCUs) blocks = 8 * kNumCUs;
        hipLaunchKernelGGL((absmax_sample_kernel<Real>), dim3((unsigned)blocks), dim3(kAbsmaxThreads), 0, stream, gout,
                           runs, (unsigned long long *)(reinterpret_cast<unsigned char *>(hdr) + 256) + 2 * kDetSlots);
        HT_LAUNCH_CHECK("forest backward (sampled magnitude bound)");
      } else if ((rc = launch_absmax<Real>(gout, pairs * d.M, &hdr->max_g, stream)) != HT_OK) {
        return rc;
      }
      // (the bound on |margin| came with the records)
      hipLaunchKernelGGL(det_scale_kernel, dim3(1), dim3(kDetFoldThreads), 0, stream, hdr, 0, double(d.S), false,
                         (const unsigned long long *)rec.bound, sampled ? kSampleGuard : 1.0, sampled);
      HT_LAUNCH_CHECK("forest backward (dW scale)");
      if (plan.parts > 1 && (rc = zero_fill(dw_fixed, size_t(d.T) * d.L * d.M * 8, stream)) != HT_OK) return rc;
    }
    if (dthr && dthr_gy > 1 && (rc = zero_fill(dthr_fixed, size_t(d.T) * d.V * 8, stream)) != HT_OK) return rc;
  }

  bool dthr_done = false;
  rc = launch_tree_kernel<Real, COMPACT, FIXED>(d, plan, w, gout, rec, dw, dw_fixed, hdr, need_c, dthr, &dthr_done, stream,
                                                gout_image);
  if (rc != HT_OK) return rc;

  if (FIXED) {
    if (dw && sampled) {
      hipLaunchKernelGGL(det_verify_kernel, dim3(1), dim3(kDetFoldThreads), 0, stream, hdr, double(d.S), kSampleGuard);
      HT_LAUNCH_CHECK("forest backward (dW bound check)");
      if (plan.parts > 1) {
        const long long n = (long long)d.T * d.L * d.M;
        hipLaunchKernelGGL(zero_if_kernel, dim3((unsigned)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096)), dim3(256),
                           0, stream, dw_fixed, n, (const int *)&hdr->redo_w);
        HT_LAUNCH_CHECK("forest backward (dW second run, clear)");
      }
      bool ignored = false;
      rc = launch_tree_kernel<Real, COMPACT, FIXED>(d, plan, w, gout, rec, dw, dw_fixed, hdr, false, (Real *)nullptr,
                                                    &ignored, stream, gout_image, true);
      if (rc != HT_OK) return rc;
    }
    if (dw) {
      if (plan.parts > 1) {
        const long long n = (long long)d.T * d.L * d.M;
        hipLaunchKernelGGL((fixed_to_real_kernel<Real>), dim3((unsigned)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096)),
                           dim3(256), 0, stream, dw_fixed, dw, n, hdr, 0);
        HT_LAUNCH_CHECK("forest backward (dW conversion)");
      }
      // non-finite magnitudes: dW by the sequential kernel instead (it does nothing unless the header says so)
      const size_t need = size_t(d.L) * d.M * sizeof(Real);
      if (need <= size_t(kLdsBytes) / 3) {
        auto kernel = det_tree_kernel<Real, true, COMPACT>;
        HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));
        hipLaunchKernelGGL(kernel, dim3((unsigned)d.T), dim3(kWave), need, stream, d, w, gout, rec, (Real *)nullptr,
                           dw, &hdr->fallback_w);
      } else {
        hipLaunchKernelGGL((det_tree_kernel<Real, false, COMPACT>), dim3((unsigned)d.T), dim3(kWave), 0, stream, d,
                           w, gout, rec, (Real *)nullptr, dw, &hdr->fallback_w);
      }
      HT_LAUNCH_CHECK("forest backward (dW fallback)");
    }
    if (need_c) {
      // the tree kernel left its bound on |c| in the header's slots
      hipLaunchKernelGGL(det_scale_kernel, dim3(1), dim3(kDetFoldThreads), 0, stream, hdr, 1,
                         double(d.S > d.T ? d.S : (long long)d.T), true, (const unsigned long long *)nullptr, 1.0, false);
      HT_LAUNCH_CHECK("forest backward (c scale)");
    }
  }

  if (dthr && !dthr_done) {
    const int vslices = int((size_t(d.V) * sizeof(double) + size_t(kLdsBytes) - 1) / size_t(kLdsBytes));
    const size_t thr_lds = size_t((d.V + vslices - 1) / vslices) * sizeof(double);
    if ((long long)d.T * vslices > 0x7fffffffLL) return fail(HT_ERR_RUNTIME, "Error: too many trees for one launch.");
    auto thr_kernel = vslices > 1 ? dthr_kernel<Real, COMPACT, FIXED, true> : dthr_kernel<Real, COMPACT, FIXED, false>;
    HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(thr_kernel)));
    hipLaunchKernelGGL(thr_kernel, dim3((unsigned)(d.T * vslices), (unsigned)dthr_gy), dim3(256), thr_lds, stream, d,
                       rec, dthr, dthr_fixed, hdr, dthr_part, dthr_gy > 1, vslices);
    HT_LAUNCH_CHECK("forest backward (dThr)");
    if (FIXED) {
      if (dthr_gy > 1) {
        const long long n = (long long)d.T * d.V;
        hipLaunchKernelGGL((fixed_to_real_kernel<Real>), dim3((unsigned)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096)),
                           dim3(256), 0, stream, dthr_fixed, dthr, n, hdr, 1);
        HT_LAUNCH_CHECK("forest backward (dThr conversion)");
      }
      const size_t need = size_t(d.V) * sizeof(Real);
      if (need <= size_t(kLdsBytes) / 3) {
        auto kernel = det_tree_kernel<Real, true, COMPACT>;
        HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));
        hipLaunchKernelGGL(kernel, dim3((unsigned)d.T), dim3(kWave), need, stream, d, w, gout, rec, dthr,
                           (Real *)nullptr, &hdr->fallback_c);
      } else {
        hipLaunchKernelGGL((det_tree_kernel<Real, false, COMPACT>), dim3((unsigned)d.T), dim3(kWave), 0, stream, d, w,
                           gout, rec, dthr, (Real *)nullptr, &hdr->fallback_c);
      }
      HT_LAUNCH_CHECK("forest backward (dThr fallback)");
    }
  }
  if (dx) {
    switch (pick_dx_tile(d.F, FIXED ? sizeof(unsigned long long) : sizeof(Real))) {
      case 64: rc = launch_dx<Real, 64, COMPACT, FIXED>(d, rec, dx, hdr, stream); break;
      case 32: rc = launch_dx<Real, 32, COMPACT, FIXED>(d, rec, dx, hdr, stream); break;
      case 16: rc = launch_dx<Real, 16, COMPACT, FIXED>(d, rec, dx, hdr, stream); break;
      case 8: rc = launch_dx<Real, 8, COMPACT, FIXED>(d, rec, dx, hdr, stream); break;
      default:  // no tile holds all features: windows of features on the smallest tile
        rc = launch_dx<Real, 8, COMPACT, FIXED>(d, rec, dx, hdr, stream);
        break;
    }
    if (rc != HT_OK) return rc;
    if (FIXED) {
      const long long blocks = (d.S + 255) / 256;
      hipLaunchKernelGGL((det_dx_kernel<Real, COMPACT>), dim3((unsigned)blocks), dim3(256), 0, stream, d, w, gout,
                         rec, dx, &hdr->fallback_c);
      HT_LAUNCH_CHECK("forest backward (dX fallback)");
    }
  }
  return rc;
}

// Sequential owner-computes pass for shapes whose accumulators do not fit LDS.
template <typename Real, bool FERN, bool COMPACT>
int backward_sequential(const ForestDims &d, const Real *x, const Node<Real> *nodes, const Real *w,
                        const Real *gout, Real *dx, Real *dthr, Real *dw, Records<Real, COMPACT> rec, bool walk,
                        hipStream_t stream) {
  int rc = HT_OK;
  if (walk && (rc = dispatch_records<Real, FERN, COMPACT>(d, x, nodes, rec, stream)) != HT_OK) return rc;
  if (dx) {
    const long long blocks = (d.S + 255) / 256;
    hipLaunchKernelGGL((det_dx_kernel<Real, COMPACT>), dim3((unsigned)blocks), dim3(256), 0, stream, d, w, gout, rec,
                       dx, (const int *)nullptr);
    HT_LAUNCH_CHECK("deterministic dX");
  }
  if (dthr || dw) {
    const size_t need = (dw ? size_t(d.L) * d.M : 0) * sizeof(Real) + (dthr ? size_t(d.V) : 0) * sizeof(Real);
    if (need <= size_t(kLdsBytes) / 3) {
      auto kernel = det_tree_kernel<Real, true, COMPACT>;
      HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));
      hipLaunchKernelGGL(kernel, dim3((unsigned)d.T), dim3(kWave), need, stream, d, w, gout, rec, dthr, dw,
                         (const int *)nullptr);
    } else {
      hipLaunchKernelGGL((det_tree_kernel<Real, false, COMPACT>), dim3((unsigned)d.T), dim3(kWave), 0, stream, d, w,
                         gout, rec, dthr, dw, (const int *)nullptr);
    }
    HT_LAUNCH_CHECK("deterministic dThr/dW");
  }
  return HT_OK;
}

// Which pipeline serves a backward call.
enum class Route { kFused, kStaged, kFixed, kSequential };

template <typename Real>
Route pick_route(const ForestDims &d, int mode, bool need_dx, bool need_dw, bool have_records) {
  if (mode == HT_BACKWARD_DETERMINISTIC)
    return staged_ok<Real>(d, need_dx, need_dw, true) ? Route::kFixed : Route::kSequential;
  if (staged_ok<Real>(d, need_dx, need_dw, false)) return (have_records || !prefer_fused(d)) ? Route::kStaged : Route::kFused;
  return have_records ? Route::kSequential : Route::kFused;  // with records there is no need to walk again
}

// Workspace after the packed vertices (stateless call) / from the start (records call): [saved records] c scratch,
// fixed-point area.
template <typename Real>
size_t route_bytes(const ForestDims &d, Route r, bool need_dthr, bool need_dw, bool have_records) {
  if (r == Route::kFused) return 0;
  size_t bytes = (have_records ? 0 : records_saved_bytes<Real>(d)) + records_scratch_bytes<Real>(d);
  if (r == Route::kFixed)
    bytes += fixed_layout(d, need_dthr, need_dw, std::is_same<Real, float>::value && compact_ok(d) && d.K == 1,
                          row_window<Real>()).total;
  return bytes;
}

template <typename Real>
int run_route(const ForestDims &d, Route route, bool fern, const Real *x, const Node<Real> *nodes, const Real *w,
              const Real *gout, Real *dx, Real *dthr, Real *dw, void *saved, void *scratch, bool walk,
              hipStream_t stream, const ImageStore *gout_image = nullptr, bool keep_c = false) {
  if (gout_image != nullptr && route != Route::kStaged)
    return fail(HT_ERR_RUNTIME, "Error: this shape cannot read the upstream gradient as an image.");
  void *fixed_ws = static_cast<unsigned char *>(scratch) + records_scratch_bytes<Real>(d);
  const bool compact = compact_ok(d);
#define HT_STAGED(FERN_, COMPACT_, FIXED_)                                                            \
  backward_staged<Real, FERN_, COMPACT_, FIXED_>(d, x, nodes, w, gout, dx, dthr, dw,                  \
                                                 carve_records<Real, COMPACT_>(d, saved, scratch), walk, fixed_ws, stream, \
                                                 gout_image, keep_c)
#define HT_SEQ(FERN_, COMPACT_)                                                                       \
  backward_sequential<Real, FERN_, COMPACT_>(d, x, nodes, w, gout, dx, dthr, dw,                      \
                                             carve_records<Real, COMPACT_>(d, saved, scratch), walk, stream)
  switch (route) {
    case Route::kFixed:
      if (fern) return compact ? HT_STAGED(true, true, true) : HT_STAGED(true, false, true);
      return compact ? HT_STAGED(false, true, true) : HT_STAGED(false, false, true);
    case Route::kSequential:
      if (fern) return compact ? HT_SEQ(true, true) : HT_SEQ(true, false);
      return compact ? HT_SEQ(false, true) : HT_SEQ(false, false);
    case Route::kStaged:
      if (fern) return compact ? HT_STAGED(true, true, false) : HT_STAGED(true, false, false);
      return compact ? HT_STAGED(false, true, false) : HT_STAGED(false, false, false);
    default:
      return fern ? dispatch_backward_fused<Real, true>(d, x, nodes, w, gout, dx, dthr, dw, stream)
                  : dispatch_backward_fused<Real, false>(d, x, nodes, w, gout, dx, dthr, dw, stream);
  }
#undef HT_STAGED
#undef HT_SEQ
}

// Clears the requested gradients as far as the route accumulates into them (the staged dX kernel overwrites all of
// dX). Returns 1 if there is nothing else to do.
template <typename Real>
int clear_gradients(const ForestDims &d, Route route, Real *dx, Real *dthr, Real *dw, hipStream_t stream, bool *done) {
  int rc;
  const bool empty = is_empty(d);
  const bool clear_dx = route != Route::kStaged || empty;
  if (dx && clear_dx && (rc = zero_fill(dx, size_t(d.S) * d.F * sizeof(Real), stream)) != HT_OK) return rc;
  // The staged atomic route stores dW and dThr from its LDS tables (every cell, by the workgroup that owns the tree)
  // unless the samples are split over several workgroups, whose shares then meet in atomics on the cleared buffers.
  bool clear_dthr = true, clear_dw = true;
  if (route == Route::kStaged && !empty) {
    TreePlan plan;
    long long dthr_part;
    int dthr_gy;
    plan_dthr(d, &dthr_part, &dthr_gy);
    if (plan_trees(d, dw != nullptr, std::is_same<Real, float>::value && compact_ok(d) && d.K == 1, &plan,
                   row_window<Real>()) &&
        plan.parts == 1) {
      clear_dw = false;
      clear_dthr = dthr_gy > 1;
    }
  }
  if (dthr && clear_dthr && (rc = zero_fill(dthr, size_t(d.T) * d.V * sizeof(Real), stream)) != HT_OK) return rc;
  if (dw && clear_dw && (rc = zero_fill(dw, size_t(d.T) * d.L * d.M * sizeof(Real), stream)) != HT_OK) return rc;
  *done = empty || (!dx && !dthr && !dw);
  return HT_OK;
}

}  // namespace

template <typename Real>
size_t forest_backward_workspace(const ForestDims &d, int mode, bool need_dx, bool need_dthr, bool need_dw) {
  if (is_empty(d)) return 0;
  const Route r = pick_route<Real>(d, mode, need_dx, need_dw, false);
  return packed_nodes_bytes<Real>(d) + route_bytes<Real>(d, r, need_dthr, need_dw, false);
}

// Whether the stateless backward can read the upstream gradient as the image of this tile geometry: atomic mode on
// the staged kernels, float data with compact records, leaf rows that tree_wide_kernel serves, and 16-byte runs that
// neither straddle a window row nor leave the image rows misaligned.
template <typename Real>
bool forest_backward_image_ok(const ForestDims &d, int mode, bool need_dx, bool need_dw, const ImageStore &img) {
  if (!std::is_same<Real, float>::value || is_empty(d) || d.K == 1 || img.nd == 0) return false;
  if (mode != HT_BACKWARD_ATOMIC || !compact_ok(d)) return false;
  if (pick_route<Real>(d, mode, need_dx, need_dw, false) != Route::kStaged) return false;
  TreePlan plan;
  if (!plan_trees(d, need_dw, false, &plan, row_window<Real>()) || !wide_rows_ok(d, plan)) return false;
  return img.win[2] % 4 == 0 && img.pad[2] % 4 == 0 && img.size[2] % 4 == 0 && img.plane % 4 == 0;
}

template <typename Real>
int forest_backward(const ForestDims &d, bool fern, const Real *x, const Real *thr, const int64_t *ord, const Real *w,
                    const Real *gout, Real *dx, Real *dthr, Real *dw, int mode, void *ws, size_t ws_bytes,
                    hipStream_t stream, const ImageStore *gout_image) {
  int rc;
  const Route route = is_empty(d) ? Route::kFused : pick_route<Real>(d, mode, dx != nullptr, dw != nullptr, false);
  if (gout_image != nullptr && !is_empty(d) && !forest_backward_image_ok<Real>(d, mode, dx != nullptr, dw != nullptr, *gout_image))
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: this shape cannot read the upstream gradient as an image.");
  bool done;
  if ((rc = clear_gradients<Real>(d, route, dx, dthr, dw, stream, &done)) != HT_OK || done) return rc;
  const size_t node_bytes = packed_nodes_bytes<Real>(d);
  const size_t need = node_bytes + route_bytes<Real>(d, route, dthr != nullptr, dw != nullptr, false);
  if (ws == nullptr || ws_bytes < need)
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: workspace too small for the backward pass.");
  unsigned char *saved = static_cast<unsigned char *>(ws) + node_bytes;
  unsigned long long *slots = route == Route::kFused ? nullptr : records_bound_slots<Real>(d, saved);
  if ((rc = pack_nodes<Real>(d, thr, ord, ws, stream, slots)) != HT_OK) return rc;
  const Node<Real> *nodes = static_cast<const Node<Real> *>(ws);
  unsigned char *scratch = saved + records_saved_bytes<Real>(d);
  return run_route<Real>(d, route, fern, x, nodes, w, gout, dx, dthr, dw, saved, scratch, true, stream, gout_image);
}

template <typename Real>
size_t forest_records_bytes(const ForestDims &d) {
  // offered where the staged kernels can consume them for every combination of requested gradients
  if (is_empty(d)) return 0;
  if (!staged_ok<Real>(d, true, true, false)) return 0;
  return records_saved_bytes<Real>(d);
}

template <typename Real>
size_t forest_backward_records_workspace(const ForestDims &d, int mode, bool need_dx, bool need_dthr, bool need_dw) {
  if (is_empty(d)) return 0;
  const Route r = pick_route<Real>(d, mode, need_dx, need_dw, true);
  return route_bytes<Real>(d, r, need_dthr, need_dw, true);
}

template <typename Real>
int forest_backward_records(const ForestDims &d, bool fern, const Real *w, const Real *gout, const void *records,
                            Real *dx, Real *dthr, Real *dw, int mode, void *ws, size_t ws_bytes,
                            hipStream_t stream) {
  int rc;
  const Route route = is_empty(d) ? Route::kFused : pick_route<Real>(d, mode, dx != nullptr, dw != nullptr, true);
  bool done;
  if ((rc = clear_gradients<Real>(d, route, dx, dthr, dw, stream, &done)) != HT_OK || done) return rc;
  const size_t need = route_bytes<Real>(d, route, dthr != nullptr, dw != nullptr, true);
  if (ws == nullptr || ws_bytes < need)
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: workspace too small for the backward pass.");
  return run_route<Real>(d, route, fern, (const Real *)nullptr, (const Node<Real> *)nullptr, w, gout, dx, dthr, dw,
                         const_cast<void *>(records), ws, false, stream);
}

// The backward pass from records for dThr / dW alone that leaves c = sign(margin) * sum_m w * g of every pair, tree
// major [T][S], at the start of the workspace: for callers inside the library that turn the records and c into an
// input-side gradient of their own instead of a dense dX. Atomic mode on the staged kernels only --
// forest_backward_keeps_c says whether a shape is served; workspace: forest_backward_records_workspace(d, atomic,
// false, true, true).
template <typename Real>
bool forest_backward_keeps_c(const ForestDims &d) {
  if (is_empty(d) || forest_records_bytes<Real>(d) == 0) return false;
  return pick_route<Real>(d, HT_BACKWARD_ATOMIC, false, true, true) == Route::kStaged;
}

template <typename Real>
int forest_backward_records_keep_c(const ForestDims &d, bool fern, const Real *w, const Real *gout, const void *records,
                                   Real *dthr, Real *dw, void *ws, size_t ws_bytes, hipStream_t stream, const Real **c) {
  int rc;
  if (!forest_backward_keeps_c<Real>(d)) return fail(HT_ERR_RUNTIME, "Error: this shape keeps no c in its workspace.");
  const Route route = Route::kStaged;
  bool done;
  if ((rc = clear_gradients<Real>(d, route, (Real *)nullptr, dthr, dw, stream, &done)) != HT_OK) return rc;
  const size_t need = route_bytes<Real>(d, route, true, true, true);
  if (ws == nullptr || ws_bytes < need)
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: workspace too small for the backward pass.");
  *c = static_cast<const Real *>(ws);
  return run_route<Real>(d, route, fern, (const Real *)nullptr, (const Node<Real> *)nullptr, w, gout, (Real *)nullptr,
                         dthr, dw, const_cast<void *>(records), ws, false, stream, nullptr, true);
}

#define HT_INSTANTIATE(Real)                                                                                          \
  template bool forest_backward_keeps_c<Real>(const ForestDims &);                                                    \
  template int forest_backward_records_keep_c<Real>(const ForestDims &, bool, const Real *, const Real *, const void *, \
                                                    Real *, Real *, void *, size_t, hipStream_t, const Real **);      \
  template size_t forest_backward_workspace<Real>(const ForestDims &, int, bool, bool, bool);                         \
  template int forest_backward<Real>(const ForestDims &, bool, const Real *, const Real *, const int64_t *,           \
                                     const Real *, const Real *, Real *, Real *, Real *, int, void *, size_t,         \
                                     hipStream_t, const ImageStore *);                                                \
  template bool forest_backward_image_ok<Real>(const ForestDims &, int, bool, bool, const ImageStore &);                                                                 \
  template size_t forest_records_bytes<Real>(const ForestDims &);                                                     \
  template size_t forest_backward_records_workspace<Real>(const ForestDims &, int, bool, bool, bool);                 \
  template int forest_backward_records<Real>(const ForestDims &, bool, const Real *, const Real *, const void *,      \
                                             Real *, Real *, Real *, int, void *, size_t, hipStream_t);
HT_INSTANTIATE(float)
HT_INSTANTIATE(double)
#undef HT_INSTANTIATE

}  // namespace ht
