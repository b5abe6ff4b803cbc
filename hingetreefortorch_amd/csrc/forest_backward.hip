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
#include "forest_tile.hpp"
#include "lds_accumulate.hpp"

namespace ht {
namespace {

constexpr int kIlp = 4;         // trees walked concurrently per thread by the records kernel
constexpr int kTreeSteps = 4;   // steps of the tree-stationary kernel whose loads are in flight together

// ---------------------------------------------------------------------------------------------------------------
// walk records
// ---------------------------------------------------------------------------------------------------------------
// COMPACT (depth <= 16 and F <= 65536): key | vertex << 16 in one word, ordinal in 16 bits.
template <typename Real, bool COMPACT>
struct Records {
  uint32_t *a;    // COMPACT: key | vertex << 16      else: key
  uint32_t *b;    // COMPACT: unused                  else: vertex
  void *ordinal;  // COMPACT: uint16_t[]              else: uint32_t[]
  Real *margin;
  Real *c;        // sign(margin) * sum_m w * g, filled by the tree kernel

  __device__ __forceinline__ void put(long long at, uint32_t key, uint32_t vertex, uint32_t ord, Real m) const {
    if (COMPACT) {
      a[at] = key | (vertex << 16);
      static_cast<uint16_t *>(ordinal)[at] = uint16_t(ord);
    } else {
      a[at] = key;
      b[at] = vertex;
      static_cast<uint32_t *>(ordinal)[at] = ord;
    }
    margin[at] = m;
  }
  __device__ __forceinline__ uint32_t key(long long at) const { return COMPACT ? (a[at] & 0xffffu) : a[at]; }
  __device__ __forceinline__ uint32_t vertex(long long at) const { return COMPACT ? (a[at] >> 16) : b[at]; }
  __device__ __forceinline__ uint32_t ord(long long at) const {
    return COMPACT ? uint32_t(static_cast<const uint16_t *>(ordinal)[at]) : static_cast<const uint32_t *>(ordinal)[at];
  }
};

static bool compact_ok(const ForestDims &d) { return d.depth <= 16 && d.F <= 65536; }

template <typename Real>
size_t records_bytes(const ForestDims &d) {
  const size_t n = size_t(d.T) * size_t(d.S);
  if (compact_ok(d)) return align_up(n * 4, 256) + align_up(n * 2, 256) + 2 * align_up(n * sizeof(Real), 256);
  return 3 * align_up(n * 4, 256) + 2 * align_up(n * sizeof(Real), 256);
}

template <typename Real, bool COMPACT>
Records<Real, COMPACT> carve_records(const ForestDims &d, void *ws) {
  const size_t n = size_t(d.T) * size_t(d.S);
  unsigned char *p = static_cast<unsigned char *>(ws);
  Records<Real, COMPACT> r;
  r.a = reinterpret_cast<uint32_t *>(p);
  p += align_up(n * 4, 256);
  r.b = nullptr;
  if (!COMPACT) {
    r.b = reinterpret_cast<uint32_t *>(p);
    p += align_up(n * 4, 256);
  }
  r.ordinal = p;
  p += align_up(n * (COMPACT ? 2 : 4), 256);
  r.margin = reinterpret_cast<Real *>(p);
  p += align_up(n * sizeof(Real), 256);
  r.c = reinterpret_cast<Real *>(p);
  return r;
}

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
  if (s >= d.S) return;
  const long long xbase = (s / d.K) * d.FK + (s % d.K);
  const int t_begin = blockIdx.y * trees_per_block;
  const int t_end = min(d.T, t_begin + trees_per_block);
  for (int tb = t_begin + tt; tb < t_end; tb += TC * kIlp) {
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
      if (t[i] < t_end)
        rec.put((long long)t[i] * d.S + s, r[i].key, r[i].vertex, uint32_t(nd[i][r[i].vertex].ord), r[i].margin);
  }
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
  HT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   int(lds)));
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
// tree-stationary dW + c
// ---------------------------------------------------------------------------------------------------------------
// grid = (tree groups, sample parts). Workgroup (g, p) owns trees [g*TB, g*TB + TB) and the samples of part p.
// LDS: dW accumulators [TB][L][M] in fp64 (if dw): the fp64 LDS atomic add is a fast hardware instruction on gfx950,
// the fp32 one is not (see lds_accumulate.hpp); each product |margin| * g is still rounded to Real first, only the
// running sum is wider.
//
// A (sample, tree) pair is served by P = M / VW adjacent lanes, lane p holding elements [p*VW, p*VW + VW) of the
// pair's M upstream-gradient values and of its leaf-weight row; a wavefront serves G = 64 / P pairs per step, pairs
// enumerated with the tree index fastest so that consecutive pairs read consecutive memory. This way every cache line
// of g and w is requested by exactly one load instruction (a thread-per-sample layout re-requests each line once per
// vector it takes out of it, and the L2 -> L1 traffic of those repeats dominated the kernel). c is reduced over the
// P lanes with shuffles.
template <typename Real, int VW, bool COMPACT>
__global__ __launch_bounds__(kForestThreads) void tree_kernel(ForestDims d, const Real *__restrict__ w,
                                                              const Real *__restrict__ gout,
                                                              Records<Real, COMPACT> rec, Real *dw, int TB,
                                                              long long part_size, bool need_c, bool dw_atomic, int P,
                                                              FastDiv div_p, int num_groups) {
  typedef Real Vec __attribute__((ext_vector_type(VW)));
  extern __shared__ __align__(16) unsigned char smem[];
  double *acc = reinterpret_cast<double *>(smem);
  // Workgroups are dealt to the 8 XCDs round robin by index, and each XCD has its own L2. Adjacent tree groups read
  // adjacent pieces of the same 128-byte lines of the upstream gradient, so they are placed on the same XCD (group =
  // (index mod 8) * groups_per_xcd + index / 8): the line is then fetched from memory once instead of once per XCD.
  const int per_xcd = (num_groups + kNumXCDs - 1) / kNumXCDs;
  const int group = int(blockIdx.x % kNumXCDs) * per_xcd + int(blockIdx.x / kNumXCDs);
  if (group >= num_groups) return;
  const int t0 = group * TB;
  const int nt = min(TB, d.T - t0);
  const long long LM = (long long)d.L * d.M;
  if (dw) {
    for (long long i = threadIdx.x; i < nt * LM; i += kForestThreads) acc[i] = 0.0;
    __syncthreads();
  }
  const long long s_begin = (long long)blockIdx.y * part_size;
  const long long s_end = min(d.S, s_begin + part_size);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  constexpr int kWaves = kForestThreads / kWave;
  const int G = kWave / P;                         // pairs per wavefront step (P <= 64)
  const int grp = div_p.div(lane), pl = lane - grp * P;
  const bool lane_on = grp < G;
  // pair q of this workgroup = (sample s_begin + q / nt, tree t0 + q % nt); a lane's q advances by kWaves * G per step
  const long long npairs = (s_end - s_begin) * nt;
  const int step = kWaves * G;
  // kTreeSteps steps are in flight together: all their record loads are issued first, then all gradient and weight
  // loads, so that a wavefront always has several independent memory round trips outstanding.
  int sub_s[kTreeSteps], sub_t[kTreeSteps];
#pragma unroll
  for (int u = 0; u < kTreeSteps; ++u) {
    sub_s[u] = (u * step) / nt;
    sub_t[u] = (u * step) - sub_s[u] * nt;
  }
  const int big = kTreeSteps * step;
  const int big_s = big / nt, big_t = big - big_s * nt;
  long long q = (long long)wave * G + grp;
  long long sl = q / nt;
  int tl = int(q - sl * nt);
  const long long row_stride = (long long)d.T * d.M;  // K == 1: distance between the gradient rows of two samples
  for (long long q0 = (long long)wave * G; q0 < npairs; q0 += big) {
    bool on[kTreeSteps];
    int tq[kTreeSteps];
    long long at[kTreeSteps], goff[kTreeSteps];
    uint32_t key[kTreeSteps];
    Real mg[kTreeSteps];
#pragma unroll
    for (int u = 0; u < kTreeSteps; ++u) {
      int tu = tl + sub_t[u];
      long long su = sl + sub_s[u];
      if (tu >= nt) {
        tu -= nt;
        ++su;
      }
      on[u] = lane_on && q + (long long)u * step < npairs;
      const long long s = s_begin + (on[u] ? su : 0);
      tq[u] = on[u] ? tu : 0;
      const int t = t0 + tq[u];
      at[u] = (long long)t * d.S + s;
      if (d.K == 1) {
        goff[u] = s * row_stride + (long long)t * d.M;
      } else {
        const long long b = s / d.K, k = s - b * d.K;
        goff[u] = ((b * d.T + t) * d.K + k) * d.M;
      }
      key[u] = rec.key(at[u]);
      mg[u] = rec.margin[at[u]];
    }
    Vec gv[kTreeSteps], wv[kTreeSteps];
#pragma unroll
    for (int u = 0; u < kTreeSteps; ++u) {
      gv[u] = *reinterpret_cast<const Vec *>(gout + goff[u] + pl * VW);
      if (need_c) wv[u] = *reinterpret_cast<const Vec *>(w + ((long long)(t0 + tq[u]) * d.L + key[u]) * d.M + pl * VW);
    }
#pragma unroll
    for (int u = 0; u < kTreeSteps; ++u) {
      if (dw && on[u]) {
        const Real a = ht_abs(mg[u]);
        double *cell = acc + (long long)tq[u] * LM + (long long)key[u] * d.M + pl * VW;
#pragma unroll
        for (int i = 0; i < VW; ++i) atomicAdd(cell + i, double(a * gv[u][i]));
      }
      if (need_c) {
        Real partial = Real(0);
#pragma unroll
        for (int i = 0; i < VW; ++i) partial += wv[u][i] * gv[u][i];
        for (int off = 1; off < P; off <<= 1) {
          const Real other = __shfl_down(partial, off, kWave);
          if (pl + off < P) partial += other;
        }
        if (on[u] && pl == 0) rec.c[at[u]] = ht_sign(mg[u]) * partial;
      }
    }
    q += big;
    sl += big_s;
    tl += big_t;
    if (tl >= nt) {
      tl -= nt;
      ++sl;
    }
  }
  if (dw) {
    __syncthreads();
    Real *dst = dw + (long long)t0 * LM;
    if (dw_atomic) {
      for (long long i = threadIdx.x; i < nt * LM; i += kForestThreads)
        if (acc[i] != 0.0) atomicAdd(dst + i, Real(acc[i]));
    } else {
      for (long long i = threadIdx.x; i < nt * LM; i += kForestThreads) dst[i] = Real(acc[i]);
    }
  }
}

// dThr[t, v] = sum over samples with selected vertex v of -c. One workgroup per tree (x sample parts).
template <typename Real, bool COMPACT>
__global__ __launch_bounds__(256) void dthr_kernel(ForestDims d, Records<Real, COMPACT> rec, Real *dthr,
                                                   long long part_size, bool use_atomic) {
  extern __shared__ __align__(16) unsigned char smem[];
  double *acc = reinterpret_cast<double *>(smem);  // fp64: fast LDS atomic, and the root vertex is a hot spot
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < d.V; i += 256) acc[i] = 0.0;
  __syncthreads();
  const long long s_begin = (long long)blockIdx.y * part_size;
  const long long s_end = min(d.S, s_begin + part_size);
  for (long long s = s_begin + threadIdx.x; s < s_end; s += 256) {
    const long long at = (long long)t * d.S + s;
    atomicAdd(acc + rec.vertex(at), -double(rec.c[at]));
  }
  __syncthreads();
  Real *dst = dthr + (long long)t * d.V;
  for (int i = threadIdx.x; i < d.V; i += 256) {
    if (use_atomic) {
      if (acc[i] != 0.0) atomicAdd(dst + i, Real(acc[i]));
    } else {
      dst[i] = Real(acc[i]);
    }
  }
}

// dX: sample tile x all trees. LDS accumulator [F][BT+1] (the pad keeps the transposing write-out conflict free).
template <typename Real, int BT, bool COMPACT>
__global__ __launch_bounds__(kForestThreads) void dx_kernel(ForestDims d, Records<Real, COMPACT> rec, Real *dx) {
  constexpr int NT = kForestThreads;
  constexpr int TC = NT / BT;
  constexpr int LD = BT + 1;
  extern __shared__ __align__(16) unsigned char smem[];
  Real *acc = reinterpret_cast<Real *>(smem);
  for (int i = threadIdx.x; i < d.F * LD; i += NT) acc[i] = Real(0);
  __syncthreads();
  const long long s0 = (long long)blockIdx.x * BT;
  const int j = threadIdx.x % BT, tt = threadIdx.x / BT;
  const long long s = s0 + j;
  if (s < d.S) {
    for (int t = tt; t < d.T; t += TC) {
      const long long at = (long long)t * d.S + s;
      lds_add(acc + rec.ord(at) * LD + j, rec.c[at]);
    }
  }
  __syncthreads();
  if (d.K == 1) {
    // dx[s, 0..F) is a contiguous row: a wavefront per sample, lanes along the features
    const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
    for (int jj = wv; jj < BT && s0 + jj < d.S; jj += NT / kWave) {
      Real *row = dx + (s0 + jj) * d.F;
      for (int f = lane; f < d.F; f += kWave) row[f] = acc[f * LD + jj];
    }
  } else {
    // dx[b, f, k]: consecutive samples of a tile are consecutive k (within one b)
    for (int i = threadIdx.x; i < d.F * BT; i += NT) {
      const int f = i / BT, jj = i - f * BT;
      const long long ss = s0 + jj;
      if (ss < d.S) dx[(ss / d.K) * d.FK + (long long)f * d.K + (ss % d.K)] = acc[f * LD + jj];
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
  HT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   int(lds)));
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
                                                     Real *dx) {
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
                                                         Real *dthr, Real *dw) {
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
struct TreePlan {
  int TB;               // trees per workgroup
  int groups, parts;    // grid
  long long part_size;  // samples per part
  size_t lds;
  int vw;               // vector width of the g / w loads
};

template <typename Real>
bool plan_trees(const ForestDims &d, bool need_dw, const Real *w, const Real *gout, TreePlan *p) {
  const size_t per_tree = size_t(d.L) * d.M * sizeof(double);
  int tb = 4;
  if (need_dw) {
    if (per_tree > size_t(kLdsBytes)) return false;
    tb = int(size_t(kLdsBytes) / per_tree);
  }
  if (tb > d.T) tb = d.T;
  // keep at least ~one workgroup per CU by shrinking the groups before splitting the samples
  while (tb > 4 && (d.T + tb - 1) / tb < kNumCUs) tb = (tb + 1) / 2;
  p->TB = tb;
  p->groups = (d.T + tb - 1) / tb;
  long long parts = 1;
  if (p->groups < kNumCUs) parts = (kNumCUs + p->groups - 1) / p->groups;
  const long long max_parts = (d.S + 4 * kForestThreads - 1) / (4 * kForestThreads);  // >= 4 samples per thread
  if (parts > max_parts) parts = max_parts;
  if (parts < 1) parts = 1;
  if (parts > 65535) parts = 65535;
  p->part_size = (d.S + parts - 1) / parts;
  p->parts = int((d.S + p->part_size - 1) / p->part_size);
  p->lds = need_dw ? size_t(tb) * per_tree : 0;
  const size_t vbytes2 = 2 * sizeof(Real), vbytes4 = 4 * sizeof(Real);
  const uintptr_t pw = reinterpret_cast<uintptr_t>(w), pg = reinterpret_cast<uintptr_t>(gout);
  p->vw = 1;
  if (d.M % 2 == 0 && pw % vbytes2 == 0 && pg % vbytes2 == 0) p->vw = 2;
  if (d.M % 4 == 0 && pw % vbytes4 == 0 && pg % vbytes4 == 0) p->vw = 4;
  return true;
}

template <typename Real, int VW, bool COMPACT>
int launch_tree_kernel(const ForestDims &d, const TreePlan &p, const Real *w, const Real *gout,
                       Records<Real, COMPACT> rec, Real *dw, bool need_c, hipStream_t stream) {
  auto kernel = tree_kernel<Real, VW, COMPACT>;
  HT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   int(p.lds)));
  const int per_xcd = (p.groups + kNumXCDs - 1) / kNumXCDs;
  hipLaunchKernelGGL(kernel, dim3((unsigned)(per_xcd * kNumXCDs), (unsigned)p.parts), dim3(kForestThreads), p.lds,
                     stream, d, w, gout, rec, dw, p.TB, p.part_size, need_c, p.parts > 1, d.M / VW,
                     FastDiv(d.M / VW), p.groups);
  HT_LAUNCH_CHECK("forest backward (trees)");
  return HT_OK;
}

template <typename Real, int BT, bool COMPACT>
int launch_dx(const ForestDims &d, Records<Real, COMPACT> rec, Real *dx, hipStream_t stream) {
  const size_t lds = size_t(d.F) * (BT + 1) * sizeof(Real);
  const long long tiles = (d.S + BT - 1) / BT;
  if (tiles > 0x7fffffffLL) return fail(HT_ERR_RUNTIME, "Error: too many sample tiles for one launch.");
  auto kernel = dx_kernel<Real, BT, COMPACT>;
  HT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   int(lds)));
  hipLaunchKernelGGL(kernel, dim3((unsigned)tiles), dim3(kForestThreads), lds, stream, d, rec, dx);
  HT_LAUNCH_CHECK("forest backward (dX)");
  return HT_OK;
}

// Largest dX tile whose padded [F][BT+1] accumulator fits LDS; 0 if none.
template <typename Real>
int pick_dx_tile(int F) {
  const int candidates[4] = {64, 32, 16, 8};
  for (int bt : candidates)
    if (size_t(F) * (bt + 1) * sizeof(Real) <= size_t(kLdsBytes)) return bt;
  return 0;
}

template <typename Real>
bool staged_ok(const ForestDims &d, bool need_dx, bool need_dw) {
  if (d.M < 1) return false;
  if (d.M > kWave) return false;  // the lanes serving one (sample, tree) pair must fit a wavefront
  if (need_dw && size_t(d.L) * d.M * sizeof(double) > size_t(kLdsBytes)) return false;
  if (size_t(d.V) * sizeof(double) > size_t(kLdsBytes)) return false;
  if (need_dx && pick_dx_tile<Real>(d.F) == 0) return false;
  return true;
}

// Problems this small finish sooner in the single fused kernel than in four launches.
static bool prefer_fused(const ForestDims &d) { return double(d.S) * double(d.T) < double(1 << 18); }

template <typename Real, bool FERN, bool COMPACT>
int backward_staged(const ForestDims &d, const Real *x, const Node<Real> *nodes, const Real *w, const Real *gout,
                    Real *dx, Real *dthr, Real *dw, void *rec_ws, hipStream_t stream) {
  Records<Real, COMPACT> rec = carve_records<Real, COMPACT>(d, rec_ws);
  int rc = dispatch_records<Real, FERN, COMPACT>(d, x, nodes, rec, stream);
  if (rc != HT_OK) return rc;
  const bool need_c = dx || dthr;
  TreePlan plan;
  if (!plan_trees<Real>(d, dw != nullptr, w, gout, &plan)) return fail(HT_ERR_RUNTIME, "Error: leaf table too large.");
  switch (plan.vw) {
    case 4: rc = launch_tree_kernel<Real, 4, COMPACT>(d, plan, w, gout, rec, dw, need_c, stream); break;
    case 2: rc = launch_tree_kernel<Real, 2, COMPACT>(d, plan, w, gout, rec, dw, need_c, stream); break;
    default: rc = launch_tree_kernel<Real, 1, COMPACT>(d, plan, w, gout, rec, dw, need_c, stream); break;
  }
  if (rc != HT_OK) return rc;
  if (dthr) {
    long long parts = d.T >= 2 * kNumCUs ? 1 : (2 * kNumCUs + d.T - 1) / d.T;
    const long long max_parts = (d.S + 1023) / 1024;
    if (parts > max_parts) parts = max_parts;
    if (parts < 1) parts = 1;
    if (parts > 65535) parts = 65535;
    const long long part_size = (d.S + parts - 1) / parts;
    const int gy = int((d.S + part_size - 1) / part_size);
    hipLaunchKernelGGL((dthr_kernel<Real, COMPACT>), dim3((unsigned)d.T, (unsigned)gy), dim3(256),
                       size_t(d.V) * sizeof(double), stream, d, rec, dthr, part_size, gy > 1);
    HT_LAUNCH_CHECK("forest backward (dThr)");
  }
  if (dx) {
    switch (pick_dx_tile<Real>(d.F)) {
      case 64: rc = launch_dx<Real, 64, COMPACT>(d, rec, dx, stream); break;
      case 32: rc = launch_dx<Real, 32, COMPACT>(d, rec, dx, stream); break;
      case 16: rc = launch_dx<Real, 16, COMPACT>(d, rec, dx, stream); break;
      default: rc = launch_dx<Real, 8, COMPACT>(d, rec, dx, stream); break;
    }
  }
  return rc;
}

template <typename Real, bool FERN, bool COMPACT>
int backward_deterministic(const ForestDims &d, const Real *x, const Node<Real> *nodes, const Real *w,
                           const Real *gout, Real *dx, Real *dthr, Real *dw, void *rec_ws, hipStream_t stream) {
  Records<Real, COMPACT> rec = carve_records<Real, COMPACT>(d, rec_ws);
  int rc = dispatch_records<Real, FERN, COMPACT>(d, x, nodes, rec, stream);
  if (rc != HT_OK) return rc;
  if (dx) {
    const long long blocks = (d.S + 255) / 256;
    hipLaunchKernelGGL((det_dx_kernel<Real, COMPACT>), dim3((unsigned)blocks), dim3(256), 0, stream, d, w, gout, rec, dx);
    HT_LAUNCH_CHECK("deterministic dX");
  }
  if (dthr || dw) {
    const size_t need = (dw ? size_t(d.L) * d.M : 0) * sizeof(Real) + (dthr ? size_t(d.V) : 0) * sizeof(Real);
    if (need <= size_t(kLdsBytes) / 3) {
      auto kernel = det_tree_kernel<Real, true, COMPACT>;
      HT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, int(need)));
      hipLaunchKernelGGL(kernel, dim3((unsigned)d.T), dim3(kWave), need, stream, d, w, gout, rec, dthr, dw);
    } else {
      hipLaunchKernelGGL((det_tree_kernel<Real, false, COMPACT>), dim3((unsigned)d.T), dim3(kWave), 0, stream, d, w,
                         gout, rec, dthr, dw);
    }
    HT_LAUNCH_CHECK("deterministic dThr/dW");
  }
  return HT_OK;
}

}  // namespace

template <typename Real>
size_t forest_backward_workspace(const ForestDims &d, int mode, bool need_dx, bool need_dthr, bool need_dw) {
  size_t bytes = packed_nodes_bytes<Real>(d);
  const bool staged = mode == HT_BACKWARD_DETERMINISTIC ||
                      (staged_ok<Real>(d, need_dx, need_dw) && !prefer_fused(d));
  (void)need_dthr;
  if (staged) bytes += records_bytes<Real>(d);
  return bytes;
}

template <typename Real>
int forest_backward(const ForestDims &d, bool fern, const Real *x, const Real *thr, const int64_t *ord, const Real *w,
                    const Real *gout, Real *dx, Real *dthr, Real *dw, int mode, void *ws, size_t ws_bytes,
                    hipStream_t stream) {
  int rc;
  const bool det = mode == HT_BACKWARD_DETERMINISTIC;
  const bool staged = det || (staged_ok<Real>(d, dx != nullptr, dw != nullptr) && !prefer_fused(d));
  // The staged dX kernel overwrites every element of dX; everything else accumulates into zeros.
  const bool empty = d.S == 0 || d.T == 0;
  const bool clear_dx = !staged || det || empty;
  if (dx && clear_dx && (rc = zero_fill(dx, size_t(d.S) * d.F * sizeof(Real), stream)) != HT_OK) return rc;
  if (dthr && (rc = zero_fill(dthr, size_t(d.T) * d.V * sizeof(Real), stream)) != HT_OK) return rc;
  if (dw && (rc = zero_fill(dw, size_t(d.T) * d.L * d.M * sizeof(Real), stream)) != HT_OK) return rc;
  if (empty || (!dx && !dthr && !dw)) return HT_OK;
  const size_t node_bytes = packed_nodes_bytes<Real>(d);
  const size_t need = node_bytes + (staged ? records_bytes<Real>(d) : 0);
  if (ws == nullptr || ws_bytes < need)
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: workspace too small for the backward pass.");
  if ((rc = pack_nodes<Real>(d, thr, ord, ws, stream)) != HT_OK) return rc;
  const Node<Real> *nodes = static_cast<const Node<Real> *>(ws);
  void *rec_ws = static_cast<unsigned char *>(ws) + node_bytes;
  const bool compact = compact_ok(d);

#define HT_CALL(fn, FERN_, COMPACT_) fn<Real, FERN_, COMPACT_>(d, x, nodes, w, gout, dx, dthr, dw, rec_ws, stream)
  if (det) {
    if (fern) return compact ? HT_CALL(backward_deterministic, true, true) : HT_CALL(backward_deterministic, true, false);
    return compact ? HT_CALL(backward_deterministic, false, true) : HT_CALL(backward_deterministic, false, false);
  }
  if (staged) {
    if (fern) return compact ? HT_CALL(backward_staged, true, true) : HT_CALL(backward_staged, true, false);
    return compact ? HT_CALL(backward_staged, false, true) : HT_CALL(backward_staged, false, false);
  }
#undef HT_CALL
  return fern ? dispatch_backward_fused<Real, true>(d, x, nodes, w, gout, dx, dthr, dw, stream)
              : dispatch_backward_fused<Real, false>(d, x, nodes, w, gout, dx, dthr, dw, stream);
}

template size_t forest_backward_workspace<float>(const ForestDims &, int, bool, bool, bool);
template size_t forest_backward_workspace<double>(const ForestDims &, int, bool, bool, bool);
template int forest_backward<float>(const ForestDims &, bool, const float *, const float *, const int64_t *,
                                    const float *, const float *, float *, float *, float *, int, void *, size_t,
                                    hipStream_t);
template int forest_backward<double>(const ForestDims &, bool, const double *, const double *, const int64_t *,
                                     const double *, const double *, double *, double *, double *, int, void *, size_t,
                                     hipStream_t);

}  // namespace ht
