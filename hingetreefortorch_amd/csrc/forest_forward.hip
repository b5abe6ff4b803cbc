// Forest / fern forward: out[b,t,k,m] = |margin| * w[t,leaf,m].
//
// A tiny pre-pass packs (threshold, ordinal) of every vertex into one aligned word pair (ordinals narrowed from the
// API's int64 and clamped into range), so a walk step costs one vertex load plus one LDS gather.
//
// One workgroup = one tile of BT samples (all features in LDS, feature major) x a range of trees. Per pass every
// thread walks TWO trees for its sample (interleaved, so the two dependent load chains overlap), parks
// (|margin|, leaf) in LDS, and then the workgroup writes the pass' outputs with the lane index running along the
// contiguous (tree, m) -- or for K > 1 the contiguous (inner position, m) -- axis of `out`, so the dominant store
// traffic is emitted as full-width rows.
#include "forest_tile.hpp"
#include "records.hpp"

namespace ht {
namespace {

template <typename Real>
__global__ __launch_bounds__(256) void pack_nodes_kernel(const Real *__restrict__ thr, const int64_t *__restrict__ ord,
                                                         Node<Real> *__restrict__ nodes, long long n, int F) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    Node<Real> v;
    v.thr = thr[i];
    v.ord = clamp_ordinal(ord[i], F);
    nodes[i] = v;
  }
}

constexpr int kOutUnroll = 5;  // output vectors per lane whose weight gathers are in flight together

// ILP = trees walked concurrently per thread; KeyT = storage type of the parked leaf keys (uint16_t up to depth 16);
// VW = outputs per lane in the output phase (divides M): the memory pipeline charges a gather instruction by its
// lanes, not by the lines it touches, so wider lanes mean proportionally fewer cycles per output.
//
// RECORD (training path): the walk results are also written out as walk records (records.hpp) for a later backward
// pass, which then does not have to walk again.
template <typename Real, bool FERN, int BT, bool XLDS, int ILP, typename KeyT, int VW, int NT, bool RECORD,
          bool COMPACT>
__global__ __launch_bounds__(NT) void forward_kernel(ForestDims d, const Real *__restrict__ x,
                                                     const Node<Real> *__restrict__ nodes,
                                                     const Real *__restrict__ w, Real *__restrict__ out,
                                                     Records<Real, COMPACT> rec, int trees_per_block,
                                                     FastDiv div_m) {
  typedef Real Vec __attribute__((ext_vector_type(VW)));
  constexpr int TC = NT / BT;        // tree slots per walk round
  constexpr int kIlp = ILP;
  constexpr int TP = TC * kIlp;      // trees per pass
  constexpr int LDR = TP + 1;        // row pitch of the per-pass results, [sample][tree]: odd, so that both the
                                     // walk's writes (lane = sample) and the output's reads (lane = tree) spread
                                     // over the LDS banks
  extern __shared__ __align__(16) unsigned char smem[];
  Real *xs = reinterpret_cast<Real *>(smem);
  Real *r_abs = xs + (XLDS ? size_t(d.F) * BT : 0);
  KeyT *r_key = reinterpret_cast<KeyT *>(r_abs + LDR * BT);

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
  for (int tb = t_begin; tb < t_end; tb += TP) {
    if (live && tb + tt < t_end) {
      const Node<Real> *nd[kIlp];
#pragma unroll
      for (int i = 0; i < kIlp; ++i) {
        const int t = min(tb + tt + i * TC, t_end - 1);  // an out-of-range slot re-walks the last tree, unused
        nd[i] = nodes + (long long)t * d.V;
      }
      WalkResult<Real> r[kIlp];
      if (XLDS)
        walk_many<Real, FERN, kIlp>(d.depth, nd, [&](int, int f) { return xs[f * BT + j]; }, r);
      else
        walk_many<Real, FERN, kIlp>(d.depth, nd, [&](int, int f) { return x[xbase + (long long)f * d.K]; }, r);
#pragma unroll
      for (int i = 0; i < kIlp; ++i) {
        r_abs[j * LDR + tt + i * TC] = ht_abs(r[i].margin);
        r_key[j * LDR + tt + i * TC] = KeyT(r[i].key);
        if (RECORD && tb + tt + i * TC < t_end)
          rec.put((long long)(tb + tt + i * TC) * d.S + s, r[i].key, r[i].vertex, r[i].ord, r[i].margin);
      }
    }
    __syncthreads();
    const int nt = min(TP, t_end - tb);
    if (d.K == 1) {
      // out[s, tb .. tb+nt, 0 .. M) is one contiguous row per sample: a wavefront per row, lanes along the row
      const int row = nt * d.M;
      const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
      constexpr int kWaves = NT / kWave;
      constexpr int WPR = kWaves > BT ? kWaves / BT : 1;  // wavefronts sharing one row
      constexpr int kStride = WPR * kWave * VW;            // elements between a lane's consecutive vectors
      const int sub = wave % WPR;
      for (int jj = wave / WPR; jj < BT; jj += kWaves / WPR) {
        const long long ss = s0 + jj;
        if (ss >= d.S) break;
        Real *orow = out + (ss * d.T + tb) * d.M;
        // kOutUnroll independent leaf-weight gathers are issued before the first store
        for (int r0 = (sub * kWave + lane) * VW; r0 < row; r0 += kStride * kOutUnroll) {
          Real a[kOutUnroll];
          Vec wv[kOutUnroll];
#pragma unroll
          for (int u = 0; u < kOutUnroll; ++u) {
            const int r = min(r0 + u * kStride, row - VW);
            const int t2 = div_m.div(r), m = r - t2 * d.M;
            const uint32_t key = r_key[jj * LDR + t2];
            a[u] = r_abs[jj * LDR + t2];
            wv[u] = *reinterpret_cast<const Vec *>(w + ((long long)(tb + t2) * d.L + key) * d.M + m);
          }
#pragma unroll
          for (int u = 0; u < kOutUnroll; ++u) {
            if (r0 + u * kStride < row) {
              Vec o;
#pragma unroll
              for (int i = 0; i < VW; ++i) o[i] = a[u] * wv[u][i];
              *reinterpret_cast<Vec *>(orow + r0 + u * kStride) = o;
            }
          }
        }
      }
    } else {
      // out[b, t, k .. , 0 .. M) is contiguous for a fixed tree
      const int row = BT * d.M, total = nt * row;
      for (int idx = threadIdx.x; idx < total; idx += NT) {
        const int t2 = idx / row, r = idx - t2 * row;
        const int jj = div_m.div(r), m = r - jj * d.M;
        const long long ss = s0 + jj;
        if (ss < d.S) {
          const uint32_t key = r_key[jj * LDR + t2];
          out[out_offset(d, ss, tb + t2, m)] = r_abs[jj * LDR + t2] * w[((long long)(tb + t2) * d.L + key) * d.M + m];
        }
      }
    }
    __syncthreads();
  }
}

template <typename Real, bool FERN, int BT, bool XLDS, int ILP, typename KeyT, int VW>
int launch_forward_rec(const ForestDims &d, const Real *x, const Node<Real> *nodes, const Real *w, Real *out,
                       void *records, hipStream_t stream);

template <typename Real, bool FERN, int BT, bool XLDS, int ILP, typename KeyT, int VW, bool RECORD, bool COMPACT>
int launch_forward_vw(const ForestDims &d, const Real *x, const Node<Real> *nodes, const Real *w, Real *out,
                      void *records, hipStream_t stream) {
  constexpr int NT = kForestThreads;
  constexpr int TP = NT / BT * ILP;
  const size_t lds = (XLDS ? size_t(d.F) * BT * sizeof(Real) : 0) + size_t(TP + 1) * BT * (sizeof(Real) + sizeof(KeyT));
  const long long tiles = (d.S + BT - 1) / BT;
  int trees_per_block, gy;
  split_trees(tiles, d.T, TP, &trees_per_block, &gy);
  if (tiles > 0x7fffffffLL) return fail(HT_ERR_RUNTIME, "Error: too many sample tiles for one launch.");
  auto kernel = forward_kernel<Real, FERN, BT, XLDS, ILP, KeyT, VW, NT, RECORD, COMPACT>;
  Records<Real, COMPACT> rec{};
  if (RECORD) rec = carve_records<Real, COMPACT>(d, records, nullptr);
  HT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   int(lds)));
  hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)gy), dim3(NT), lds, stream, d, x, nodes, w, out, rec,
                     trees_per_block, FastDiv(d.M));
  HT_LAUNCH_CHECK("forest forward");
  return HT_OK;
}

template <typename Real, bool FERN, int BT, bool XLDS, int ILP, typename KeyT, int VW>
int launch_forward_rec(const ForestDims &d, const Real *x, const Node<Real> *nodes, const Real *w, Real *out,
                       void *records, hipStream_t stream) {
  if (!records)
    return launch_forward_vw<Real, FERN, BT, XLDS, ILP, KeyT, VW, false, true>(d, x, nodes, w, out, records, stream);
  if (compact_ok(d))
    return launch_forward_vw<Real, FERN, BT, XLDS, ILP, KeyT, VW, true, true>(d, x, nodes, w, out, records, stream);
  return launch_forward_vw<Real, FERN, BT, XLDS, ILP, KeyT, VW, true, false>(d, x, nodes, w, out, records, stream);
}

template <typename Real, bool FERN, int BT, bool XLDS, int ILP, typename KeyT>
int launch_forward_as(const ForestDims &d, const Real *x, const Node<Real> *nodes, const Real *w, Real *out,
                      void *records, hipStream_t stream) {
  // widest output vector that M and the pointers allow (K > 1 keeps scalar outputs)
  const uintptr_t pw = reinterpret_cast<uintptr_t>(w), po = reinterpret_cast<uintptr_t>(out);
  if (d.K == 1 && d.M % 4 == 0 && pw % (4 * sizeof(Real)) == 0 && po % (4 * sizeof(Real)) == 0)
    return launch_forward_rec<Real, FERN, BT, XLDS, ILP, KeyT, 4>(d, x, nodes, w, out, records, stream);
  if (d.K == 1 && d.M % 2 == 0 && pw % (2 * sizeof(Real)) == 0 && po % (2 * sizeof(Real)) == 0)
    return launch_forward_rec<Real, FERN, BT, XLDS, ILP, KeyT, 2>(d, x, nodes, w, out, records, stream);
  return launch_forward_rec<Real, FERN, BT, XLDS, ILP, KeyT, 1>(d, x, nodes, w, out, records, stream);
}

// Four trees per thread with 16-bit parked keys where the depth allows it, else two trees with 32-bit keys: both keep
// the per-pass results of a 1024-thread workgroup under the LDS left beside a 128 KB sample tile.
template <typename Real, bool FERN, int BT, bool XLDS>
int launch_forward(const ForestDims &d, const Real *x, const Node<Real> *nodes, const Real *w, Real *out,
                   void *records, hipStream_t stream) {
  if (d.depth <= 16) return launch_forward_as<Real, FERN, BT, XLDS, 4, uint16_t>(d, x, nodes, w, out, records, stream);
  return launch_forward_as<Real, FERN, BT, XLDS, 2, uint32_t>(d, x, nodes, w, out, records, stream);
}

template <typename Real, bool FERN>
int dispatch_forward(const ForestDims &d, const Real *x, const Node<Real> *nodes, const Real *w, Real *out,
                     void *records, hipStream_t stream) {
  // room for the per-pass results: (4 trees x 1024 threads + one pad column) x (|margin| + key)
  const size_t reserve = size_t(4) * kForestThreads * (sizeof(Real) + sizeof(uint32_t));
  int bt = pick_tile<Real>(d.F, reserve);
  // With many outputs per leaf the output phase dominates, and it runs better on a narrower tile: twice the trees per
  // pass (longer contiguous row segments per store burst, half the barriers) and one row per wavefront.
  if (d.M >= 8 && bt >= 32) bt /= 2;
  switch (bt) {
    case 64: return launch_forward<Real, FERN, 64, true>(d, x, nodes, w, out, records, stream);
    case 32: return launch_forward<Real, FERN, 32, true>(d, x, nodes, w, out, records, stream);
    case 16: return launch_forward<Real, FERN, 16, true>(d, x, nodes, w, out, records, stream);
    case 8: return launch_forward<Real, FERN, 8, true>(d, x, nodes, w, out, records, stream);
    default: return launch_forward<Real, FERN, 64, false>(d, x, nodes, w, out, records, stream);
  }
}

}  // namespace

template <typename Real>
size_t packed_nodes_bytes(const ForestDims &d) {
  return align_up(size_t(d.T) * d.V * sizeof(Node<Real>), 256);
}

template <typename Real>
int pack_nodes(const ForestDims &d, const Real *thr, const int64_t *ord, void *dst, hipStream_t stream) {
  const long long n = (long long)d.T * d.V;
  if (n == 0) return HT_OK;
  hipLaunchKernelGGL(pack_nodes_kernel<Real>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, thr, ord,
                     static_cast<Node<Real> *>(dst), n, d.F);
  HT_LAUNCH_CHECK("pack vertices");
  return HT_OK;
}

template <typename Real>
size_t forest_forward_workspace(const ForestDims &d) {
  return packed_nodes_bytes<Real>(d);
}

template <typename Real>
int forest_forward(const ForestDims &d, bool fern, const Real *x, const Real *thr, const int64_t *ord, const Real *w,
                   Real *out, void *records, void *ws, size_t ws_bytes, hipStream_t stream) {
  if (d.S == 0 || d.T == 0) return HT_OK;
  if (ws == nullptr || ws_bytes < packed_nodes_bytes<Real>(d))
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: workspace too small for the forward pass.");
  int rc = pack_nodes<Real>(d, thr, ord, ws, stream);
  if (rc != HT_OK) return rc;
  const Node<Real> *nodes = static_cast<const Node<Real> *>(ws);
  return fern ? dispatch_forward<Real, true>(d, x, nodes, w, out, records, stream)
              : dispatch_forward<Real, false>(d, x, nodes, w, out, records, stream);
}

#define HT_INSTANTIATE(Real)                                                                                          \
  template size_t packed_nodes_bytes<Real>(const ForestDims &);                                                       \
  template int pack_nodes<Real>(const ForestDims &, const Real *, const int64_t *, void *, hipStream_t);              \
  template size_t forest_forward_workspace<Real>(const ForestDims &);                                                 \
  template int forest_forward<Real>(const ForestDims &, bool, const Real *, const Real *, const int64_t *,            \
                                    const Real *, Real *, void *, void *, size_t, hipStream_t);
HT_INSTANTIATE(float)
HT_INSTANTIATE(double)
#undef HT_INSTANTIATE

}  // namespace ht
