// Forest / fern forward: out[b,t,k,m] = |margin| * w[t,leaf,m].
//
// A tiny pre-pass packs (threshold, ordinal) of every vertex into one aligned word pair (ordinals narrowed from the
// API's int64 and clamped into range), so a walk step costs one vertex load plus one LDS gather.
//
// One workgroup = one tile of BT samples (all features in LDS, feature major) x a range of trees. Two kernels:
//   forward_rows_kernel  (K == 1, the common case) every wavefront walks and writes on its own, see below;
//   forward_kernel       (any K) per pass every thread walks several trees for its sample, parks (|margin|, leaf) in
//                        LDS, and then the workgroup writes the pass' outputs with the lane index running along the
//                        contiguous (tree, m) -- or for K > 1 the contiguous (inner position, m) -- axis of `out`.
#include <type_traits>

#include "forest_tile.hpp"
#include "records.hpp"

namespace ht {
namespace {

template <typename Real>
__global__ __launch_bounds__(256) void pack_nodes_kernel(const Real *__restrict__ thr, const int64_t *__restrict__ ord,
                                                         Node<Real> *__restrict__ nodes, long long n, int F,
                                                         unsigned long long *zero_slots) {
  if (zero_slots && blockIdx.x == 0)
    for (int k = threadIdx.x; k < kBoundSlots; k += 256) zero_slots[k] = 0ull;
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
                                                     FastDiv div_m, ImageStore img, FeatureNorm<Real> norm) {
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
    load_tile<Real, BT, NT>(xs, x, d, s0, norm);
    __syncthreads();
  }
  const int j = threadIdx.x % BT, tt = threadIdx.x / BT;
  const long long s = s0 + j;
  const bool live = s < d.S;
  const long long xbase = live ? (s / d.K) * d.FK + (s % d.K) : 0;
  const bool normalise = norm.mean != nullptr;

  const int t_begin = blockIdx.y * trees_per_block;
  const int t_end = min(d.T, t_begin + trees_per_block);
  MarginBits margin_bound;  // RECORD: bound on the |margin| this lane recorded
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
        walk_many<Real, FERN, kIlp>(
            d.depth, nd,
            [&](int, int f) {
              const Real v = x[xbase + (long long)f * d.K];
              return normalise ? (v - norm.mean[f]) * norm.rstd[f] : v;
            },
            r);
#pragma unroll
      for (int i = 0; i < kIlp; ++i) {
        r_abs[j * LDR + tt + i * TC] = ht_abs(r[i].margin);
        r_key[j * LDR + tt + i * TC] = KeyT(r[i].key);
        if (RECORD && tb + tt + i * TC < t_end) {
          rec.put((long long)(tb + tt + i * TC) * d.S + s, r[i].key, r[i].vertex, r[i].ord, r[i].margin);
          margin_bound.take(r[i].margin);
        }
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
    } else if (d.K >= BT) {
      // Inner data dimensions: for a fixed tree the rows of consecutive inner positions follow each other,
      // out[b, t, k .. k + BT, 0 .. M) -- one contiguous run per tree unless the tile crosses into the next batch
      // row, which moves the rest of the run by (T - 1) * K * M elements. Lanes run along (position, m) in vectors
      // of VW elements; the tree is uniform per pass of the loop, so its part of every address is scalar.
      const long long b0 = s0 / d.K;
      const int k0 = int(s0 - b0 * d.K);
      const long long wrap = (long long)(d.T - 1) * d.K * d.M;
      const int vecs = BT * d.M / VW;  // per tree
      for (int t2 = 0; t2 < nt; ++t2) {
        Real *obase = out + ((b0 * d.T + tb + t2) * d.K + k0) * d.M;
        const Real *wbase = w + (long long)(tb + t2) * d.L * d.M;
        for (int v = threadIdx.x; v < vecs; v += NT) {
          const int r = v * VW;
          const int jj = div_m.div(r), m = r - jj * d.M;
          if (s0 + jj >= d.S) continue;
          Real *dst = obase + r + (k0 + jj >= d.K ? wrap : 0ll);
          if (img.nd) {
            // the vector's VW outputs are consecutive along the innermost window dimension, hence in the image
            const bool next = k0 + jj >= d.K;
            const long long at = img.offset(k0 + jj - (next ? d.K : 0), m);
            if (at < 0) continue;
            dst = out + ((b0 + (next ? 1 : 0)) * d.T + tb + t2) * img.plane + at;
          }
          const uint32_t key = r_key[jj * LDR + t2];
          const Real a = r_abs[jj * LDR + t2];
          const Vec wv = *reinterpret_cast<const Vec *>(wbase + (long long)key * d.M + m);
          Vec o;
#pragma unroll
          for (int i = 0; i < VW; ++i) o[i] = a * wv[i];
          *reinterpret_cast<Vec *>(dst) = o;
        }
      }
    } else {
      // inner dimensions shorter than the tile: generic addressing
      const int row = BT * d.M, total = nt * row;
      for (int idx = threadIdx.x; idx < total; idx += NT) {
        const int t2 = idx / row, r = idx - t2 * row;
        const int jj = div_m.div(r), m = r - jj * d.M;
        const long long ss = s0 + jj;
        if (ss < d.S) {
          long long at = out_offset(d, ss, tb + t2, m);
          if (img.nd) {
            const long long b = ss / d.K;
            const long long in_plane = img.offset(int(ss - b * d.K), m);
            if (in_plane < 0) continue;
            at = (b * d.T + tb + t2) * img.plane + in_plane;
          }
          const uint32_t key = r_key[jj * LDR + t2];
          out[at] = r_abs[jj * LDR + t2] * w[((long long)(tb + t2) * d.L + key) * d.M + m];
        }
      }
    }
    __syncthreads();
  }
  if (RECORD) bound_publish(margin_bound_value<Real>(margin_bound.bits), rec.bound, (blockIdx.y * gridDim.x + blockIdx.x) % unsigned(kBoundSlots));
}


// ---------------------------------------------------------------------------------------------------------------
// row kernel (K == 1): wavefront-autonomous walk + output
// ---------------------------------------------------------------------------------------------------------------
// Two-level vertices ("quads") of a float tree whose ordinals fit 10 bits: the vertex of an even level together with
// its two children in one 16-byte word, so a walk costs one vector load per TWO levels. The vector memory pipeline
// charges a divergent load per instruction and per distinct line, not per byte, which makes this the cheapest form
// of the data-dependent vertex stream. Quads of level pair k (levels 2k, 2k+1) start at (4^k - 1) / 3; quad i of a
// pair holds vertex (2^(2k) - 1) + i and its grandchildren are quads 4i .. 4i+3 of the next pair.
struct __align__(16) QuadNode {
  float thr, thr_left, thr_right;
  uint32_t ords;  // ordinal | left ordinal << 10 | right ordinal << 20
};
constexpr int kQuadOrdinalBits = 10;

static inline long long quads_per_tree(int depth) {
  long long n = 0, level = 1;
  for (int l = 0; l < depth; l += 2) {
    n += level;
    level *= 4;
  }
  return n;
}

__global__ __launch_bounds__(256) void pack_quads_kernel(const float *__restrict__ thr, const int64_t *__restrict__ ord,
                                                         QuadNode *__restrict__ quads, int T, int V, int NQ, int F,
                                                         unsigned long long *zero_slots) {
  if (zero_slots && blockIdx.x == 0)
    for (int k = threadIdx.x; k < kBoundSlots; k += 256) zero_slots[k] = 0ull;
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long long)T * NQ) return;
  const int t = int(i / NQ), q = int(i - (long long)t * NQ);
  int k = 0, base = 0, width = 1;
  while (q >= base + width) {
    base += width;
    width *= 4;
    ++k;
  }
  const long long v = ((1ll << (2 * k)) - 1) + (q - base);
  const float *th = thr + (long long)t * V;
  const int64_t *od = ord + (long long)t * V;
  QuadNode n;
  n.thr = th[v];
  uint32_t o = uint32_t(clamp_ordinal(od[v], F));
  n.thr_left = n.thr_right = 0.f;
  if (2 * v + 2 < V) {
    n.thr_left = th[2 * v + 1];
    n.thr_right = th[2 * v + 2];
    o |= uint32_t(clamp_ordinal(od[2 * v + 1], F)) << kQuadOrdinalBits;
    o |= uint32_t(clamp_ordinal(od[2 * v + 2], F)) << (2 * kQuadOrdinalBits);
  }
  n.ords = o;
  quads[i] = n;
}

constexpr int kTopQuads = 5;  // quads of the first two level pairs (levels 0..3): 1 + 4

// N interleaved walks over quads; xs_j = this lane's column of the feature-major sample tile (pitch BT).
// TOP_LDS: top[i] is an LDS copy of the first kTopQuads quads of walk i's tree; levels 0..3 are then read from LDS
// (the same for all samples of a tree slot: broadcasts), which takes two of the five dependent memory round trips
// out of a depth-10 walk.
//
// The walk is bound by its vector instructions, so a level is kept to the few that the semantics need: the decisions
// are shifted into `path` through the carry of one add (path = 2 * path + (margin > 0): most significant bit first,
// which is also the index of the current vertex inside its level), the running minimum is the signed margin itself
// (compared by magnitude; the root seeds it, so a NaN root sticks as in the reference, HingeTreeCommon.h:157-178),
// and beside it only the level and ordinal of the minimum are carried, packed in one word. The leaf key (decision of
// level i in bit i) is the bit reversal of the finished path, the selected vertex is rebuilt from the path and the
// level. TRACK = false (no walk records wanted) carries |margin| alone: r.margin is then the magnitude, r.vertex and
// r.ord are 0.
template <int N, int BT, bool TOP_LDS, bool TRACK>
__device__ __forceinline__ void walk_quads(int depth, const QuadNode *const (&quads)[N],
                                           const QuadNode *const (&top)[N], const float *xs_j,
                                           WalkResult<float> (&r)[N]) {
  uint32_t path[N], info[N];  // info: ordinal | level << kQuadOrdinalBits of the smallest |margin| so far
  float best[N];              // TRACK: its signed margin; else its magnitude
  constexpr uint32_t kMask = (1u << kQuadOrdinalBits) - 1;
#pragma unroll
  for (int i = 0; i < N; ++i) path[i] = 0, info[i] = 0, best[i] = 0.f;
  float root[N];
  uint32_t base = 0, width = 1;  // first quad / number of quads of the current level pair
  auto take = [&](int i, float m, uint32_t ord, int lvl) {
    if (TRACK) {
      const bool closer = ht_abs(m) < ht_abs(best[i]);
      best[i] = closer ? m : best[i];
      info[i] = closer ? (ord | (uint32_t(lvl) << kQuadOrdinalBits)) : info[i];
    } else {
      best[i] = __builtin_fminf(best[i], ht_abs(m));  // a NaN margin never wins; a NaN root is put back below
    }
  };
  for (int lvl = 0; lvl < depth; lvl += 2) {
    QuadNode n[N];
    if (TOP_LDS && lvl < 4) {
#pragma unroll
      for (int i = 0; i < N; ++i) n[i] = top[i][base + path[i]];
    } else {
#pragma unroll
      for (int i = 0; i < N; ++i) n[i] = quads[i][base + path[i]];
    }
    float m0[N];
#pragma unroll
    for (int i = 0; i < N; ++i) m0[i] = xs_j[(n[i].ords & kMask) * BT] - n[i].thr;
    const bool two = lvl + 1 < depth;
    float m1[N];
    uint32_t o1[N];
    bool right0[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
      right0[i] = m0[i] > 0.f;
      const float t1 = right0[i] ? n[i].thr_right : n[i].thr_left;
      o1[i] = (n[i].ords >> (right0[i] ? 2 * kQuadOrdinalBits : kQuadOrdinalBits)) & kMask;
      m1[i] = two ? xs_j[o1[i] * BT] - t1 : 0.f;
    }
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if (lvl == 0) {
        root[i] = m0[i];
        best[i] = TRACK ? m0[i] : ht_abs(m0[i]);
        info[i] = n[i].ords & kMask;
      } else {
        take(i, m0[i], n[i].ords & kMask, lvl);
      }
      path[i] = path[i] + path[i] + (right0[i] ? 1u : 0u);
      if (two) {
        take(i, m1[i], o1[i], lvl + 1);
        path[i] = path[i] + path[i] + ((m1[i] > 0.f) ? 1u : 0u);
      }
    }
    base += width;
    width *= 4u;
  }
#pragma unroll
  for (int i = 0; i < N; ++i) {
    r[i].key = __brev(path[i]) >> (32 - depth);
    if (TRACK) {
      const uint32_t lvl = info[i] >> kQuadOrdinalBits;
      r[i].vertex = ((1u << lvl) - 1u) + (path[i] >> (uint32_t(depth) - lvl));
      r[i].ord = info[i] & kMask;
      r[i].margin = best[i];
    } else {
      r[i].vertex = 0;
      r[i].ord = 0;
      r[i].margin = (root[i] != root[i]) ? root[i] : best[i];
    }
  }
}

// N interleaved fern walks whose vertices are staged in LDS level major: walk i's vertex of level l is
// mine[l * TPW + i * STRIDE]. Like walk_quads the loop carries the path (decisions, most significant bit first), the
// signed margin of the smallest |margin| so far (seeded by level 0, strict '<' afterwards: HingeTreeCommon.h:72-91) and
// one word holding that level and its ordinal; TRACK = false carries |margin| alone. A fern's selected vertex is its
// level.
template <typename Real, int N, int BT, int STRIDE, int TPW, bool TRACK>
__device__ __forceinline__ void walk_ferns_staged(int depth, const Node<Real> *mine, const Real *xs_j,
                                                  WalkResult<Real> (&r)[N]) {
  constexpr int kLevelShift = 24;  // ordinals index a tile in LDS: far below 2^24
  uint32_t path[N], info[N];
  Real best[N], root[N];
#pragma unroll
  for (int i = 0; i < N; ++i) path[i] = 0, info[i] = 0, best[i] = Real(0), root[i] = Real(0);
  // (Issuing the reads of several levels together -- a fern's vertices do not depend on the path -- was measured and
  // gained nothing: 0.470 against 0.471 ms for the fern benchmark's forward.)
  auto level = [&](int lvl, auto first_tag) {
    constexpr bool FIRST = decltype(first_tag)::value;
    Node<Real> n[N];
#pragma unroll
    for (int i = 0; i < N; ++i) n[i] = mine[lvl * TPW + i * STRIDE];
    Real m[N];
#pragma unroll
    for (int i = 0; i < N; ++i) m[i] = xs_j[int(n[i].ord) * BT] - n[i].thr;
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if (FIRST) {
        root[i] = m[i];
        best[i] = TRACK ? m[i] : ht_abs(m[i]);
        info[i] = uint32_t(n[i].ord);
      } else if (TRACK) {
        const bool closer = ht_abs(m[i]) < ht_abs(best[i]);
        best[i] = closer ? m[i] : best[i];
        info[i] = closer ? (uint32_t(n[i].ord) | (uint32_t(lvl) << kLevelShift)) : info[i];
      } else {
        const Real a = ht_abs(m[i]);
        best[i] = (a < best[i]) ? a : best[i];  // a NaN margin never wins; a NaN root is put back below
      }
      path[i] = path[i] + path[i] + ((m[i] > Real(0)) ? 1u : 0u);
    }
  };
  level(0, std::true_type{});
  for (int lvl = 1; lvl < depth; ++lvl) level(lvl, std::false_type{});
#pragma unroll
  for (int i = 0; i < N; ++i) {
    r[i].key = __brev(path[i]) >> (32 - depth);
    if (TRACK) {
      r[i].vertex = info[i] >> kLevelShift;
      r[i].ord = info[i] & ((1u << kLevelShift) - 1u);
      r[i].margin = best[i];
    } else {
      r[i].vertex = 0;
      r[i].ord = 0;
      r[i].margin = (root[i] != root[i]) ? root[i] : best[i];
    }
  }
}

// What lane + 1 of the wavefront holds in v (lane 63: 0): one data-parallel move of the vector ALU per 32 bits.
__device__ __forceinline__ float value_of_next_lane(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x130 /* wave_shl:1 */, 0xf, 0xf, false));
}
__device__ __forceinline__ double value_of_next_lane(double v) {
  const long long b = __double_as_longlong(v);
  const int lo = __builtin_amdgcn_update_dpp(0, int(uint32_t(b)), 0x130, 0xf, 0xf, false);
  const int hi = __builtin_amdgcn_update_dpp(0, int(uint32_t(uint64_t(b) >> 32)), 0x130, 0xf, 0xf, false);
  return __longlong_as_double((long long)((uint64_t(uint32_t(hi)) << 32) | uint32_t(lo)));
}

constexpr int kRowIlp = 4;     // trees walked concurrently per lane
constexpr int kRowUnroll = 5;  // output vectors per lane whose weight gathers are in flight together

// One step of a wavefront of the row kernels: this lane's sample (column xs_j of the tile) through the kRowIlp trees
// tb + slot + i * SLOTS of the step's TPW = SLOTS * kRowIlp trees. stage_area is the wavefront's own piece of LDS (BT *
// (TPW + 1) values), free while the walks run: the top quads of the step's trees (QUAD) or the vertices of its ferns
// are copied there once per step. TRACK: also the selected vertex, its ordinal and the signed margin.
template <typename Real, bool FERN, bool QUAD, int BT, bool TRACK>
__device__ __forceinline__ void rows_walk_step(const ForestDims &d, const void *__restrict__ vertices, int NQ, int tb,
                                               int t_end, int slot, int lane, const Real *xs_j, Real *stage_area,
                                               WalkResult<Real> (&r)[kRowIlp]) {
  constexpr int SLOTS = kWave / BT;
  constexpr int TPW = SLOTS * kRowIlp;
  constexpr int LDP = TPW + 1;
  int t[kRowIlp];
#pragma unroll
  for (int i = 0; i < kRowIlp; ++i) t[i] = min(tb + slot + i * SLOTS, t_end - 1);  // surplus slots re-walk, unused
  if constexpr (QUAD) {
    const QuadNode *all = static_cast<const QuadNode *>(vertices);
    const QuadNode *qn[kRowIlp];
#pragma unroll
    for (int i = 0; i < kRowIlp; ++i) qn[i] = all + (long long)t[i] * NQ;
    // The top of every tree is the same for all samples: the wavefront copies the first quads of its TPW trees
    // into LDS once per step (into the space of the parked results, which nobody reads before this step's walks
    // are over), where they fit.
    constexpr bool kTopFits = size_t(TPW) * kTopQuads * sizeof(QuadNode) <= size_t(BT) * LDP * sizeof(Real);
    if (kTopFits && NQ >= kTopQuads) {
      QuadNode *stage = reinterpret_cast<QuadNode *>(stage_area);
      for (int i = lane; i < TPW * kTopQuads; i += kWave) {
        const int tt = i / kTopQuads, q = i - tt * kTopQuads;
        stage[i] = all[(long long)min(tb + tt, t_end - 1) * NQ + q];
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      const QuadNode *top[kRowIlp];
#pragma unroll
      for (int i = 0; i < kRowIlp; ++i) top[i] = stage + (slot + i * SLOTS) * kTopQuads;
      walk_quads<kRowIlp, BT, true, TRACK>(d.depth, qn, top, xs_j, r);
      // every lane has read its quads before any lane overwrites them with results
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    } else {
      walk_quads<kRowIlp, BT, false, TRACK>(d.depth, qn, qn, xs_j, r);
    }
  } else {
    const Node<Real> *all = static_cast<const Node<Real> *>(vertices);
    bool staged = false;
    if constexpr (FERN) {
      // A fern's vertex is the same for every sample, so a vector load of it would fetch one address per tree
      // slot and still cost a full trip through the vector memory pipeline per level. Instead the wavefront
      // copies the vertices of its TPW ferns into LDS once per step -- into the space of the parked results,
      // which nobody reads before this step's walks are over -- and the walk reads them as LDS broadcasts.
      Node<Real> *stage = reinterpret_cast<Node<Real> *>(stage_area);
      if (size_t(TPW) * d.depth * sizeof(Node<Real>) <= size_t(BT) * LDP * sizeof(Real)) {
        staged = true;
        // level major, [level][fern]: the ferns of a lane's kRowIlp walks then lie a compile-time distance apart
        for (int i = lane; i < TPW * d.depth; i += kWave) {
          const int lv = i / TPW, tt = i - lv * TPW;
          stage[i] = all[(long long)min(tb + tt, t_end - 1) * d.V + lv];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        walk_ferns_staged<Real, kRowIlp, BT, SLOTS, TPW, TRACK>(d.depth, stage + slot, xs_j, r);
        // every lane has read its vertices before any lane overwrites them with results
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
      }
    }
    if (!staged) {
      const Node<Real> *nd[kRowIlp];
#pragma unroll
      for (int i = 0; i < kRowIlp; ++i) nd[i] = all + (long long)t[i] * d.V;
      walk_many<Real, FERN, kRowIlp>(d.depth, nd, [&](int, int f) { return xs_j[f * BT]; }, r);
    }
  }
}

// One workgroup = one tile of BT samples (all features in LDS, feature major) x a range of trees, like
// forward_kernel, but every wavefront works on its own: lanes = BT samples x 64/BT tree slots, each lane walks
// kRowIlp trees, parks (|margin|, leaf) in a wavefront-private piece of LDS, and the same wavefront then writes the
// TPW = 64/BT * kRowIlp trees' outputs of its samples, lanes running along the contiguous (tree, m) axis of a row.
// There is no workgroup barrier after the tile load, so at any moment some wavefronts of a CU walk (vertex gathers)
// while others store, and the two phases overlap instead of alternating across the whole device.
//
// QUAD selects two-level vertices (float trees, F <= 1024); otherwise Node<Real> is walked level by level.
// GW = elements per weight gather and per store (divides M). RECORD: also write the walk records.
// ODD (with GW = 2): an odd number of outputs per leaf written as pairs all the same. A sample's run of a step's trees
// starts on an even element, so the pairs (e, e + 1), e even, are aligned stores; the leaf table is a padded copy whose
// odd trees' rows are shifted by one element, which makes a pair's first element an even index of its row in every
// tree: one aligned gather per pair, (M + 1) / 2 gather slots per tree instead of M (the cost of the output phase is
// its number of gather instructions, and its stores must leave no holes for a later instruction to fill).
// Needs an even tree count, so that every sample's row of the output starts on an even element.
template <typename Real, bool FERN, bool QUAD, int BT, int GW, bool ODD, bool RECORD, bool COMPACT>
__global__ __launch_bounds__(kForestThreads) void forward_rows_kernel(ForestDims d, const Real *__restrict__ x,
                                                                      const void *__restrict__ vertices, int NQ,
                                                                      const Real *__restrict__ w,
                                                                      Real *__restrict__ out,
                                                                      Records<Real, COMPACT> rec,
                                                                      int trees_per_block, FastDiv div_m,
                                                                      FastDiv div_u_full, int wpitch) {
  typedef Real Vec __attribute__((ext_vector_type(GW)));
  constexpr int NT = kForestThreads;
  constexpr int kWaves = NT / kWave;
  constexpr int SLOTS = kWave / BT;        // tree slots of a wavefront
  constexpr int TPW = SLOTS * kRowIlp;     // trees per wavefront step
  constexpr int LDP = TPW + 1;             // odd pitch of the parked results, [sample][tree]
  extern __shared__ __align__(16) unsigned char smem[];
  Real *xs = reinterpret_cast<Real *>(smem);
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  Real *p_abs = xs + size_t(d.F) * BT + size_t(wave) * (BT * LDP);
  uint16_t *p_key = reinterpret_cast<uint16_t *>(xs + size_t(d.F) * BT + size_t(kWaves) * (BT * LDP)) +
                    size_t(wave) * (BT * LDP);

  const long long s0 = (long long)blockIdx.x * BT;
  load_tile<Real, BT, NT>(xs, x, d, s0);
  __syncthreads();

  const int j = lane % BT, slot = lane / BT;
  const long long s = s0 + j;
  const bool live = s < d.S;
  const int n_live = int(min<long long>(BT, d.S - s0));
  const Real *xs_j = xs + j;
  const int t_begin = blockIdx.y * trees_per_block;
  const int t_end = min(d.T, t_begin + trees_per_block);
  const uint32_t TM = uint32_t(d.T) * uint32_t(d.M);
  MarginBits margin_bound;  // RECORD: bound on the |margin| this lane recorded
  // Single-output rows: a wavefront step's run of a sample is TPW * 4 bytes, half a 64-byte sector or less, and the
  // other half is written by another wavefront at another time. Streaming stores send each half to memory by itself
  // (the fern benchmark wrote 922 MB for 786 MB); ordinary stores let the L2 put the halves together first (forward
  // 0.458 -> 0.430 ms there). Wider rows fill their sectors and stream (ordinary stores: 0.89 -> 1.39 ms at 10 outputs).
  const bool narrow_rows = d.M == 1;
  auto store_out = [&](Vec v, Real *at) {
    if (GW == 1 && narrow_rows)
      *reinterpret_cast<Vec *>(at) = v;
    else
      __builtin_nontemporal_store(v, reinterpret_cast<Vec *>(at));
  };

  // Output phase, lane constants of burst slot q for `un` slots per burst and u vectors per sample: where the parked
  // walk result of the vector's pair lies, the vector's column in the leaf table of the step's first tree, and its
  // offset in the output from the step's first element.
  auto burst_constants = [&](auto un_tag, int u_per_sample, FastDiv by_u, uint32_t *park, uint32_t *wcol,
                             uint32_t *off) {
#pragma unroll
    for (int q = 0; q < decltype(un_tag)::value; ++q) {
      const int u = lane + q * kWave;
      const int jj = by_u.div(u);
      const int e = (u - jj * u_per_sample) * GW;
      const int tt = div_m.div(e), m = e - tt * d.M;
      park[q] = uint32_t(jj * LDP + tt);
      wcol[q] = uint32_t(tt) * uint32_t(d.L) * uint32_t(wpitch) + uint32_t(m);
      off[q] = uint32_t(jj) * TM + uint32_t(e);
    }
  };
  // ... prepared once for the complete steps of a complete tile
  uint32_t full_park[kRowUnroll], full_wcol[kRowUnroll], full_off[kRowUnroll];
  int full_un = 0;
  {
    const int u_full = TPW * d.M / GW, total_full = BT * u_full;
    if (!ODD && n_live == BT) {
      if (total_full % (kWave * kRowUnroll) == 0 && (kWave * kRowUnroll) % u_full == 0) full_un = kRowUnroll;
    }
#pragma unroll
    for (int q = 0; q < kRowUnroll; ++q) full_park[q] = full_wcol[q] = full_off[q] = 0;
    if (full_un == kRowUnroll)
      burst_constants(std::integral_constant<int, kRowUnroll>{}, u_full, div_u_full, full_park, full_wcol, full_off);
  }

  // ODD: what this lane does in every instruction of the output phase (see there)
  constexpr int kOddUnroll = 4;
  int odd_upi = 1, odd_unit = 0, odd_second = 0, odd_idx = 0, odd_role = 0;
  bool odd_active = false;
  uint32_t odd_park[kOddUnroll] = {}, odd_wcol[kOddUnroll] = {}, odd_off[kOddUnroll] = {};
  if (ODD) {
    const int slots = d.M + 1, hs = slots >> 1;
    odd_upi = kWave / slots;                 // pairs of trees per wavefront instruction
    odd_unit = lane / slots;
    const int r = lane - odd_unit * slots;   // 0 .. M: the gather slot inside the pair of trees
    odd_active = odd_unit < odd_upi;
    odd_second = r >= hs ? 1 : 0;            // the odd tree of the pair
    odd_idx = odd_second ? 2 * (r - hs) : 2 * r;  // first element read, as an index of its (shifted) row
    odd_role = r == hs - 1 ? 1 : (r == hs ? 2 : 0);  // 1: the even tree's last element; 2: the odd tree's first
    // complete steps of a complete tile, kOddUnroll instructions per iteration: an iteration is then a whole number of
    // samples (kOddUnroll is a multiple of the TPW / 2 pairs of trees of a sample's run wherever BT >= 32), and
    // what changes from one iteration to the next is the sample alone
#pragma unroll
    for (int q = 0; q < kOddUnroll; ++q) {
      const int g = q * odd_upi + odd_unit, jj = g / (TPW / 2), tt = 2 * (g - jj * (TPW / 2)) + odd_second;
      odd_park[q] = uint32_t(jj * LDP + tt);
      odd_wcol[q] = uint32_t(tt) * uint32_t(d.L) * uint32_t(wpitch) + uint32_t(odd_idx);
      odd_off[q] = uint32_t(jj) * TM + uint32_t(tt * d.M + odd_idx - odd_second);
    }
  }

  for (int tb = t_begin + wave * TPW; tb < t_end; tb += kWaves * TPW) {
    // ---- walk: this lane's sample through trees tb + slot + i * SLOTS
    {
      __builtin_amdgcn_s_setprio(0);
      WalkResult<Real> r[kRowIlp];
      rows_walk_step<Real, FERN, QUAD, BT, RECORD>(d, vertices, NQ, tb, t_end, slot, lane, xs_j, p_abs, r);
#pragma unroll
      for (int i = 0; i < kRowIlp; ++i) {
        const Real a = ht_abs(r[i].margin);
        p_abs[j * LDP + slot + i * SLOTS] = a;
        p_key[j * LDP + slot + i * SLOTS] = uint16_t(r[i].key);
        if (RECORD && live && tb + slot + i * SLOTS < t_end)
          rec.put((long long)(tb + slot + i * SLOTS) * d.S + s, r[i].key, r[i].vertex, r[i].ord, r[i].margin);
        // (surplus slots re-walk an existing tree and dead lanes a zero row of the tile: their margins may join the
        // bound, which then costs no predicate)
        if (RECORD) margin_bound.take_abs(a);
      }
    }
    // the parked results are read by other lanes of this wavefront only
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // ---- output: out[s0 + jj, tb .. tb + nt, 0 .. M) is one contiguous run per sample
    // A wavefront in this phase issues few instructions and waits on memory in between; with the higher priority its
    // gathers and stores are issued as soon as their operands are there instead of queueing behind the walks of the
    // SIMD's other wavefronts (forward at 65536 x 1024 features, 1000 trees of depth 10, 10 outputs: 0.958 -> 0.931 ms;
    // the opposite order of priorities changes nothing).
    __builtin_amdgcn_s_setprio(3);
    const int nt = min(TPW, t_end - tb);
    Real *obase = out + ((long long)s0 * d.T + tb) * d.M;
    const Real *wbase = w + (long long)tb * d.L * wpitch;  // wpitch: elements between leaf rows (M, or padded)
    if constexpr (ODD) {
      // nt is even here (the tree count is, and so is every step's first tree). Two trees are M + 1 gathers: the even
      // tree's pairs (0,1) .. (M-3,M-2), its last element alone, the odd tree's first element alone, its pairs (1,2) ..
      // (M-2,M-1) -- each one aligned 8-byte gather from the padded (and, in odd trees, shifted) rows. The two
      // lone elements are neighbours in the output: the lane of the first fetches the second's product from the next
      // lane and stores the pair, the lane of the second stores nothing. A wavefront instruction serves whole pairs
      // of trees (64 / (M + 1) of them), so what a lane does is the same in every instruction and the two lone
      // elements always sit in neighbouring lanes.
      const int units = nt >> 1, total_units = n_live * units;
      if ((kOddUnroll % (TPW / 2)) == 0 && nt == TPW && n_live == BT) {
        uint32_t park[kOddUnroll], off[kOddUnroll];
        int g[kOddUnroll];
#pragma unroll
        for (int q = 0; q < kOddUnroll; ++q) park[q] = odd_park[q], off[q] = odd_off[q], g[q] = q * odd_upi + odd_unit;
        const int per_iteration = odd_upi * kOddUnroll;               // pairs of trees
        const uint32_t samples = uint32_t(per_iteration / (TPW / 2));  // ... which are whole samples
        for (int g0 = 0; g0 < total_units; g0 += per_iteration) {
          Real a[kOddUnroll];
          Vec wv[kOddUnroll];
          bool live_q[kOddUnroll];
#pragma unroll
          for (int q = 0; q < kOddUnroll; ++q) {
            live_q[q] = odd_active && g[q] < total_units;
            const uint32_t at = live_q[q] ? park[q] : 0u;  // idle lanes read a parked result that exists
            const uint32_t key = p_key[at];
            a[q] = p_abs[at];
            wv[q] = *reinterpret_cast<const Vec *>(wbase + key * uint32_t(wpitch) + odd_wcol[q]);
          }
#pragma unroll
          for (int q = 0; q < kOddUnroll; ++q) {
            Vec o;
            o[0] = a[q] * wv[q][0];
            o[1] = a[q] * wv[q][1];
            const Real from_next = value_of_next_lane(o[1]);
            if (odd_role == 1) o[1] = from_next;
            if (live_q[q] && odd_role != 2) store_out(o, obase + off[q]);
            park[q] += samples * LDP;
            off[q] += samples * TM;
            g[q] += per_iteration;
          }
        }
        __builtin_amdgcn_wave_barrier();
        continue;
      }
      const FastDiv by_units = nt == TPW ? FastDiv(TPW / 2) : FastDiv(units);  // (the first: a constant)
      for (int g0 = 0; g0 < total_units; g0 += odd_upi * kRowUnroll) {
        Real a[kRowUnroll];
        Vec wv[kRowUnroll], o[kRowUnroll];
        uint32_t off[kRowUnroll];
        bool live_q[kRowUnroll];
#pragma unroll
        for (int q = 0; q < kRowUnroll; ++q) {
          const int g = g0 + q * odd_upi + odd_unit;
          live_q[q] = odd_active && g < total_units;
          const int gc = min(g, total_units - 1);
          const int jj = by_units.div(gc), tt = 2 * (gc - jj * units) + odd_second;
          const uint32_t key = p_key[jj * LDP + tt];
          a[q] = p_abs[jj * LDP + tt];
          wv[q] = *reinterpret_cast<const Vec *>(wbase + (uint32_t(tt) * uint32_t(d.L) + key) * uint32_t(wpitch) +
                                                 odd_idx);
          off[q] = uint32_t(jj) * TM + uint32_t(tt * d.M + odd_idx - odd_second);
        }
#pragma unroll
        for (int q = 0; q < kRowUnroll; ++q) {
          o[q][0] = a[q] * wv[q][0];
          o[q][1] = a[q] * wv[q][1];
        }
#pragma unroll
        for (int q = 0; q < kRowUnroll; ++q) {
          const Real from_next = value_of_next_lane(o[q][1]);
          if (odd_role == 1) o[q][1] = from_next;
          // (ordinary stores for the pairs in sectors that the step's run covers only in part -- an odd run of 8 M
          // elements is not a whole number of 64-byte sectors -- were measured and cost 15 %)
          if (live_q[q] && odd_role != 2) store_out(o[q], obase + off[q]);
        }
      }
      __builtin_amdgcn_wave_barrier();
      continue;
    }
    const int U = nt * d.M / GW;  // vectors per sample
    FastDiv div_u = div_u_full;   // divisor TPW * M / GW, prepared by the host
    if (nt != TPW) div_u = FastDiv(U);
    const int total = n_live * U;
    // Whole bursts, and a burst is a whole number of samples: which tree and output a lane serves in slot q of a
    // burst is the same in every burst, so the divisions are done once (complete tiles of the benchmark shapes: 32
    // samples x 8 trees x 10 outputs = 4 bursts of 5 vectors per lane, 8 samples each) and a burst only advances the
    // sample. For complete steps of a complete tile the lane constants were even prepared before the loop over the
    // steps. (A four-vector burst for one output per leaf, whose step is 256 vectors, was measured slower than the
    // general loop below: ferns 0.464 -> 0.485 ms.)
    auto bursts = [&](auto un_tag, const uint32_t *park0, const uint32_t *wcol0, const uint32_t *off0) {
      constexpr int UN = decltype(un_tag)::value;
      constexpr int kBurst = kWave * UN;  // vectors a wavefront handles per iteration
      uint32_t park[UN], wcol[UN], off[UN];
#pragma unroll
      for (int q = 0; q < UN; ++q) park[q] = park0[q], wcol[q] = wcol0[q], off[q] = off0[q];
      const uint32_t park_step = uint32_t(kBurst / U) * LDP, off_step = uint32_t(kBurst / U) * TM;
      for (int burst = 0; burst < total; burst += kBurst) {
        Real a[UN];
        Vec wv[UN];
#pragma unroll
        for (int q = 0; q < UN; ++q) {
          const uint32_t key = p_key[park[q]];
          a[q] = p_abs[park[q]];
          wv[q] = *reinterpret_cast<const Vec *>(wbase + key * uint32_t(wpitch) + wcol[q]);
        }
#pragma unroll
        for (int q = 0; q < UN; ++q) {
          Vec o;
#pragma unroll
          for (int i = 0; i < GW; ++i) o[i] = a[q] * wv[q][i];
          store_out(o, obase + off[q]);
          park[q] += park_step;
          off[q] += off_step;
        }
      }
    };
    if (full_un != 0 && nt == TPW) {
      bursts(std::integral_constant<int, kRowUnroll>{}, full_park, full_wcol, full_off);
    } else if (total % (kWave * kRowUnroll) == 0 && (kWave * kRowUnroll) % U == 0) {
      uint32_t park[kRowUnroll], wcol[kRowUnroll], off[kRowUnroll];
      burst_constants(std::integral_constant<int, kRowUnroll>{}, U, div_u, park, wcol, off);
      bursts(std::integral_constant<int, kRowUnroll>{}, park, wcol, off);
    } else {
      for (int u0 = lane; u0 < total; u0 += kWave * kRowUnroll) {
        Real a[kRowUnroll];
        Vec wv[kRowUnroll];
        uint32_t off[kRowUnroll];
#pragma unroll
        for (int q = 0; q < kRowUnroll; ++q) {
          const int u = min(u0 + q * kWave, total - 1);
          const int jj = div_u.div(u);
          const int e = (u - jj * U) * GW;
          const int tt = div_m.div(e), m = e - tt * d.M;
          const uint32_t key = p_key[jj * LDP + tt];
          a[q] = p_abs[jj * LDP + tt];
          wv[q] = *reinterpret_cast<const Vec *>(wbase + (uint32_t(tt) * uint32_t(d.L) + key) * uint32_t(wpitch) + m);
          off[q] = uint32_t(jj) * TM + uint32_t(e);
        }
#pragma unroll
        for (int q = 0; q < kRowUnroll; ++q) {
          if (u0 + q * kWave < total) {
            Vec o;
#pragma unroll
            for (int i = 0; i < GW; ++i) o[i] = a[q] * wv[q][i];
            // streaming store: the output is written once and not read here, so it should not displace the vertices
            // and leaf weights that the gathers keep re-reading from L2 (measured: 1.45 -> 1.17 ms at the headline
            // shape)
            store_out(o, obase + off[q]);
          }
        }
      }
    }
    // the next step's parking writes follow this step's reads in program order; the LDS serves a wavefront's
    // requests in order
    __builtin_amdgcn_wave_barrier();
  }
  if (RECORD) bound_publish(margin_bound_value<Real>(margin_bound.bits), rec.bound, (blockIdx.y * gridDim.x + blockIdx.x) % unsigned(kBoundSlots));
}

// The walk of forward_rows_kernel without its output phase, for the maps: a wavefront parks one or two values per
// (sample, tree) pair of its step and writes them with its lanes running along the tree axis of [S][T], so that a
// sample's values of the step's TPW trees leave as one run (the int64 leaf keys of 8 trees are a whole 64-byte sector).
// MARGIN = false: leaf keys, as int64 [S][T] (leafmap) and / or as 16-bit keys tree major [T][S] (keys16, what the
// reachability histogram reads; stored by the walking lane itself, whose neighbours hold the neighbouring samples).
// MARGIN = true: signed margins [S][T] and the selected ordinals as int64 [S][T].
template <typename Real, bool FERN, bool QUAD, int BT, bool MARGIN>
__global__ __launch_bounds__(kForestThreads) void maps_rows_kernel(ForestDims d, const Real *__restrict__ x,
                                                                   const void *__restrict__ vertices, int NQ,
                                                                   int64_t *__restrict__ leafmap,
                                                                   uint16_t *__restrict__ keys16,
                                                                   Real *__restrict__ margins,
                                                                   int64_t *__restrict__ ordinals,
                                                                   int trees_per_block) {
  constexpr int NT = kForestThreads;
  constexpr int kWaves = NT / kWave;
  constexpr int SLOTS = kWave / BT;
  constexpr int TPW = SLOTS * kRowIlp;
  constexpr int LDP = TPW + 1;
  extern __shared__ __align__(16) unsigned char smem[];
  Real *xs = reinterpret_cast<Real *>(smem);
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  Real *p_val = xs + size_t(d.F) * BT + size_t(wave) * (BT * LDP);
  uint16_t *p_u16 = reinterpret_cast<uint16_t *>(xs + size_t(d.F) * BT + size_t(kWaves) * (BT * LDP)) +
                    size_t(wave) * (BT * LDP);
  const long long s0 = (long long)blockIdx.x * BT;
  load_tile<Real, BT, NT>(xs, x, d, s0);
  __syncthreads();
  const int j = lane % BT, slot = lane / BT;
  const long long s = s0 + j;
  const bool live = s < d.S;
  const int n_live = int(min<long long>(BT, d.S - s0));
  const Real *xs_j = xs + j;
  const int t_begin = blockIdx.y * trees_per_block;
  const int t_end = min(d.T, t_begin + trees_per_block);
  for (int tb = t_begin + wave * TPW; tb < t_end; tb += kWaves * TPW) {
    {
      WalkResult<Real> r[kRowIlp];
      rows_walk_step<Real, FERN, QUAD, BT, MARGIN>(d, vertices, NQ, tb, t_end, slot, lane, xs_j, p_val, r);
#pragma unroll
      for (int i = 0; i < kRowIlp; ++i) {
        const int at = j * LDP + slot + i * SLOTS;
        if (MARGIN) {
          p_val[at] = r[i].margin;
          p_u16[at] = uint16_t(r[i].ord);
        } else {
          p_u16[at] = uint16_t(r[i].key);
          const int t = tb + slot + i * SLOTS;
          if (keys16 && live && t < t_end) keys16[(long long)t * d.S + s] = uint16_t(r[i].key);
        }
      }
    }
    // the parked values are read by other lanes of this wavefront only
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int nt = min(TPW, t_end - tb);
    const int total = n_live * nt;
    const FastDiv by_nt(nt);
    const long long base = s0 * d.T + tb;
    if (MARGIN || leafmap) {
      for (int u = lane; u < total; u += kWave) {
        const int jj = nt == TPW ? u / TPW : by_nt.div(u);
        const int tt = u - jj * nt;
        const long long at = base + (long long)jj * d.T + tt;
        if (MARGIN) {
          if (margins) __builtin_nontemporal_store(p_val[jj * LDP + tt], margins + at);
          if (ordinals) __builtin_nontemporal_store((long long)p_u16[jj * LDP + tt], reinterpret_cast<long long *>(ordinals) + at);
        } else {
          __builtin_nontemporal_store((long long)p_u16[jj * LDP + tt], reinterpret_cast<long long *>(leafmap) + at);
        }
      }
    }
    // the next step's parking writes follow this step's reads in program order
    __builtin_amdgcn_wave_barrier();
  }
}

template <typename Real>
static inline size_t rows_lds_bytes(int F, int bt) {
  const int tpw = kWave / bt * kRowIlp;
  return size_t(F) * bt * sizeof(Real) +
         size_t(kForestThreads / kWave) * bt * (tpw + 1) * (sizeof(Real) + sizeof(uint16_t));
}

template <typename Real>
static inline int pick_rows_tile(int F) {
  const int candidates[4] = {64, 32, 16, 8};
  for (int bt : candidates)
    if (rows_lds_bytes<Real>(F, bt) <= size_t(kLdsBytes)) return bt;
  return 0;
}

// Shapes the row kernel serves: contiguous rows (K == 1), 16-bit parked keys, 32-bit element offsets inside a
// wavefront step, and a sample tile that fits LDS.
template <typename Real>
static inline bool rows_ok(const ForestDims &d) {
  if (d.K != 1 || d.depth > 16 || d.M < 1) return false;
  if ((long long)d.T * d.M * 64 >= (1ll << 31)) return false;
  if ((long long)kWave * kRowIlp * d.L * d.M >= (1ll << 31)) return false;
  return pick_rows_tile<Real>(d.F) != 0;
}

template <typename Real>
static inline bool quads_ok(const ForestDims &d, bool fern) {
  return std::is_same<Real, float>::value && !fern && d.F <= (1 << kQuadOrdinalBits) &&
         (long long)d.T * quads_per_tree(d.depth) < (1ll << 31);
}

template <typename Real, bool FERN, bool QUAD, int BT, int GW, bool ODD, bool RECORD, bool COMPACT>
int launch_rows(const ForestDims &d, const Real *x, const void *vertices, const Real *w, int wpitch, Real *out,
                void *records, hipStream_t stream) {
  constexpr int TPW = kWave / BT * kRowIlp;
  constexpr int TP = kForestThreads / kWave * TPW;
  const size_t lds = rows_lds_bytes<Real>(d.F, BT);
  const long long tiles = (d.S + BT - 1) / BT;
  int trees_per_block, gy;
  split_trees(tiles, d.T, TP, &trees_per_block, &gy);
  if (tiles > 0x7fffffffLL) return fail(HT_ERR_RUNTIME, "Error: too many sample tiles for one launch.");
  auto kernel = forward_rows_kernel<Real, FERN, QUAD, BT, GW, ODD, RECORD, COMPACT>;
  Records<Real, COMPACT> rec{};
  if (RECORD) rec = carve_records<Real, COMPACT>(d, records, nullptr);
  HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));
  hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)gy), dim3(kForestThreads), lds, stream, d, x, vertices,
                     int(quads_per_tree(d.depth)), w, out, rec, trees_per_block, FastDiv(d.M),
                     FastDiv(TPW * d.M / GW), wpitch);
  HT_LAUNCH_CHECK("forest forward (rows)");
  return HT_OK;
}

template <typename Real, bool FERN, bool QUAD, int BT, int GW, bool ODD = false>
int launch_rows_rec(const ForestDims &d, const Real *x, const void *vertices, const Real *w, int wpitch, Real *out,
                    void *records, hipStream_t stream) {
  if (!records)
    return launch_rows<Real, FERN, QUAD, BT, GW, ODD, false, true>(d, x, vertices, w, wpitch, out, records, stream);
  if (compact_ok(d))
    return launch_rows<Real, FERN, QUAD, BT, GW, ODD, true, true>(d, x, vertices, w, wpitch, out, records, stream);
  return launch_rows<Real, FERN, QUAD, BT, GW, ODD, true, false>(d, x, vertices, w, wpitch, out, records, stream);
}

template <typename Real, bool FERN, bool QUAD, int BT>
int launch_rows_gw(const ForestDims &d, const Real *x, const void *vertices, const Real *w, int wpitch, bool shifted,
                   Real *out, void *records, hipStream_t stream) {
  const uintptr_t pw = reinterpret_cast<uintptr_t>(w), po = reinterpret_cast<uintptr_t>(out);
  if (shifted)  // odd rows in pairs: the table was laid out for it and the alignments were checked, see odd_pairs_ok
    return launch_rows_rec<Real, FERN, QUAD, BT, 2, true>(d, x, vertices, w, wpitch, out, records, stream);
  if (d.M % 4 == 0 && wpitch % 4 == 0 && pw % (4 * sizeof(Real)) == 0 && po % (4 * sizeof(Real)) == 0)
    return launch_rows_rec<Real, FERN, QUAD, BT, 4>(d, x, vertices, w, wpitch, out, records, stream);
  if (d.M % 2 == 0 && wpitch % 2 == 0 && pw % (2 * sizeof(Real)) == 0 && po % (2 * sizeof(Real)) == 0)
    return launch_rows_rec<Real, FERN, QUAD, BT, 2>(d, x, vertices, w, wpitch, out, records, stream);
  return launch_rows_rec<Real, FERN, QUAD, BT, 1>(d, x, vertices, w, wpitch, out, records, stream);
}

template <typename Real, bool FERN, bool QUAD>
int dispatch_rows(const ForestDims &d, const Real *x, const void *vertices, const Real *w, int wpitch, bool shifted,
                  Real *out, void *records, hipStream_t stream) {
  switch (pick_rows_tile<Real>(d.F)) {
    case 64: return launch_rows_gw<Real, FERN, QUAD, 64>(d, x, vertices, w, wpitch, shifted, out, records, stream);
    case 32: return launch_rows_gw<Real, FERN, QUAD, 32>(d, x, vertices, w, wpitch, shifted, out, records, stream);
    case 16: return launch_rows_gw<Real, FERN, QUAD, 16>(d, x, vertices, w, wpitch, shifted, out, records, stream);
    default: return launch_rows_gw<Real, FERN, QUAD, 8>(d, x, vertices, w, wpitch, shifted, out, records, stream);
  }
}

template <typename Real, bool FERN, int BT, bool XLDS, int ILP, typename KeyT, int VW>
int launch_forward_rec(const ForestDims &d, const Real *x, const Node<Real> *nodes, const Real *w, Real *out,
                       void *records, hipStream_t stream, const ImageStore &img, const FeatureNorm<Real> &norm);

template <typename Real, bool FERN, int BT, bool XLDS, int ILP, typename KeyT, int VW, bool RECORD, bool COMPACT>
int launch_forward_vw(const ForestDims &d, const Real *x, const Node<Real> *nodes, const Real *w, Real *out,
                      void *records, hipStream_t stream, const ImageStore &img, const FeatureNorm<Real> &norm) {
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
  HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));
  hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)gy), dim3(NT), lds, stream, d, x, nodes, w, out, rec,
                     trees_per_block, FastDiv(d.M), img, norm);
  HT_LAUNCH_CHECK("forest forward");
  return HT_OK;
}

template <typename Real, bool FERN, int BT, bool XLDS, int ILP, typename KeyT, int VW>
int launch_forward_rec(const ForestDims &d, const Real *x, const Node<Real> *nodes, const Real *w, Real *out,
                       void *records, hipStream_t stream, const ImageStore &img, const FeatureNorm<Real> &norm) {
  if (!records)
    return launch_forward_vw<Real, FERN, BT, XLDS, ILP, KeyT, VW, false, true>(d, x, nodes, w, out, records, stream,
                                                                               img, norm);
  if (compact_ok(d))
    return launch_forward_vw<Real, FERN, BT, XLDS, ILP, KeyT, VW, true, true>(d, x, nodes, w, out, records, stream,
                                                                              img, norm);
  return launch_forward_vw<Real, FERN, BT, XLDS, ILP, KeyT, VW, true, false>(d, x, nodes, w, out, records, stream, img,
                                                                             norm);
}

template <typename Real, bool FERN, int BT, bool XLDS, int ILP, typename KeyT>
int launch_forward_as(const ForestDims &d, const Real *x, const Node<Real> *nodes, const Real *w, Real *out,
                      void *records, hipStream_t stream, const ImageStore &img, const FeatureNorm<Real> &norm) {
  // widest output vector that M and the pointers allow (inner dimensions shorter than the tile keep scalar outputs);
  // into an image, a vector must also stay inside one window row and keep the image rows aligned
  const uintptr_t pw = reinterpret_cast<uintptr_t>(w), po = reinterpret_cast<uintptr_t>(out);
  const bool runs = d.K == 1 || d.K >= BT;  // the branches of the kernel that store whole vectors
  auto fits = [&](int vw) {
    if (!runs || d.M % vw != 0 || pw % (vw * sizeof(Real)) != 0 || po % (vw * sizeof(Real)) != 0) return false;
    return img.nd == 0 || (img.win[2] % vw == 0 && img.pad[2] % vw == 0 && img.size[2] % vw == 0);
  };
  if (fits(4))
    return launch_forward_rec<Real, FERN, BT, XLDS, ILP, KeyT, 4>(d, x, nodes, w, out, records, stream, img, norm);
  if (fits(2))
    return launch_forward_rec<Real, FERN, BT, XLDS, ILP, KeyT, 2>(d, x, nodes, w, out, records, stream, img, norm);
  return launch_forward_rec<Real, FERN, BT, XLDS, ILP, KeyT, 1>(d, x, nodes, w, out, records, stream, img, norm);
}

// Four trees per thread with 16-bit parked keys where the depth allows it, else two trees with 32-bit keys: both keep
// the per-pass results of a 1024-thread workgroup under the LDS left beside a 128 KB sample tile.
template <typename Real, bool FERN, int BT, bool XLDS>
int launch_forward(const ForestDims &d, const Real *x, const Node<Real> *nodes, const Real *w, Real *out,
                   void *records, hipStream_t stream, const ImageStore &img, const FeatureNorm<Real> &norm) {
  if (d.depth <= 16)
    return launch_forward_as<Real, FERN, BT, XLDS, 4, uint16_t>(d, x, nodes, w, out, records, stream, img, norm);
  return launch_forward_as<Real, FERN, BT, XLDS, 2, uint32_t>(d, x, nodes, w, out, records, stream, img, norm);
}

template <typename Real, bool FERN>
int dispatch_forward(const ForestDims &d, const Real *x, const Node<Real> *nodes, const Real *w, Real *out,
                     void *records, hipStream_t stream, const ImageStore &img, const FeatureNorm<Real> &norm) {
  // room for the per-pass results: (4 trees x 1024 threads + one pad column) x (|margin| + key)
  const size_t reserve = size_t(4) * kForestThreads * (sizeof(Real) + sizeof(uint32_t));
  int bt = pick_tile<Real>(d.F, reserve);
  // With many outputs per leaf the output phase dominates, and it runs better on a narrower tile: twice the trees per
  // pass (longer contiguous row segments per store burst, half the barriers) and one row per wavefront.
  if (d.M >= 8 && bt >= 32) bt /= 2;
  switch (bt) {
    case 64: return launch_forward<Real, FERN, 64, true>(d, x, nodes, w, out, records, stream, img, norm);
    case 32: return launch_forward<Real, FERN, 32, true>(d, x, nodes, w, out, records, stream, img, norm);
    case 16: return launch_forward<Real, FERN, 16, true>(d, x, nodes, w, out, records, stream, img, norm);
    case 8: return launch_forward<Real, FERN, 8, true>(d, x, nodes, w, out, records, stream, img, norm);
    default: return launch_forward<Real, FERN, 64, false>(d, x, nodes, w, out, records, stream, img, norm);
  }
}

}  // namespace

template <typename Real>
size_t packed_nodes_bytes(const ForestDims &d) {
  return align_up(size_t(d.T) * d.V * sizeof(Node<Real>), 256);
}

template <typename Real>
int pack_nodes(const ForestDims &d, const Real *thr, const int64_t *ord, void *dst, hipStream_t stream,
               unsigned long long *zero_slots) {
  const long long n = (long long)d.T * d.V;
  if (n == 0) return HT_OK;
  hipLaunchKernelGGL(pack_nodes_kernel<Real>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, thr, ord,
                     static_cast<Node<Real> *>(dst), n, d.F, zero_slots);
  HT_LAUNCH_CHECK("pack vertices");
  return HT_OK;
}

template <typename Real>
static size_t quads_bytes(const ForestDims &d) {
  return align_up(size_t(d.T) * size_t(quads_per_tree(d.depth)) * sizeof(QuadNode), 256);
}

// Leaf rows of M values are gathered at random; a row that straddles two 64-byte sectors costs two requests to L2,
// and the rate of those requests per CU is what bounds the row kernel. So where a row is not already a whole number
// of sectors (or a power-of-two fraction of one), the forward pass first copies the leaf table to a pitch that is:
// M = 10 floats -> 16. Worth it only when the gathers outnumber the table rows by far.
template <typename Real>
static int weight_pitch(const ForestDims &d) {
  constexpr int kSector = 64 / int(sizeof(Real));
  int p = d.M;
  if (d.M <= kSector) {
    p = 1;
    while (p < d.M) p <<= 1;
  } else {
    p = (d.M + kSector - 1) / kSector * kSector;
  }
  if (p == d.M || !rows_ok<Real>(d)) return d.M;
  if (d.S < 8ll * d.L || (long long)kWave * kRowIlp * d.L * p >= (1ll << 31)) return d.M;
  if (size_t(d.T) * d.L * p * sizeof(Real) > (size_t(1) << 30)) return d.M;
  return p;
}

template <typename Real>
static size_t vertex_bytes(const ForestDims &d) {
  const size_t nodes = packed_nodes_bytes<Real>(d);
  const size_t quads = (quads_ok<Real>(d, false) && rows_ok<Real>(d)) ? quads_bytes<Real>(d) : 0;
  return nodes > quads ? nodes : quads;
}

template <typename Real>
size_t forest_forward_workspace(const ForestDims &d) {
  if (is_empty(d)) return 0;
  const int p = weight_pitch<Real>(d);
  return vertex_bytes<Real>(d) + (p != d.M ? align_up(size_t(d.T) * d.L * p * sizeof(Real), 256) : 0);
}

// An odd number (> 1) of outputs per leaf goes out in pairs where every sample's row of the output starts on an even
// element (even tree count), the output is aligned for pairs, and the leaf table is copied to an even pitch with room
// for the shift of the odd trees' rows.
template <typename Real>
static bool odd_pairs_ok(const ForestDims &d, int wpitch, const Real *out) {
  return d.M > 1 && (d.M & 1) && d.M + 1 <= kWave / 2 && (d.T & 1) == 0 && wpitch != d.M && wpitch % 2 == 0 && wpitch >= d.M + 1 &&
         reinterpret_cast<uintptr_t>(out) % (2 * sizeof(Real)) == 0;
}

// shift_odd (with L = rows per tree): the rows of odd trees start at element 1 of their pitch, see forward_rows_kernel.
template <typename Real>
__global__ __launch_bounds__(256) void pad_rows_kernel(const Real *__restrict__ w, Real *__restrict__ dst, long long rows,
                                                       int M, int P, bool shift_odd, int L) {
  const long long n = rows * P;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
    const long long r = i / P;
    const int m = int(i - r * P) - ((shift_odd && ((r / L) & 1)) ? 1 : 0);
    dst[i] = (m >= 0 && m < M) ? w[r * M + m] : Real(0);
  }
}

// The same copy for a power-of-two pitch and an even row length: one thread per pair of elements, index arithmetic by
// shifts, one store per thread over a flat grid (the form in which plain stores run fastest).
template <typename Real>
__global__ __launch_bounds__(256) void pad_rows_pairs_kernel(const Real *__restrict__ w, Real *__restrict__ dst,
                                                             long long pairs, int M, int log2_pairs_per_row) {
  typedef Real Vec2 __attribute__((ext_vector_type(2)));
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= pairs) return;
  const long long r = i >> log2_pairs_per_row;
  const int m = int(i - (r << log2_pairs_per_row)) * 2;
  Vec2 v = {Real(0), Real(0)};
  if (m < M) v = *reinterpret_cast<const Vec2 *>(w + r * M + m);
  *reinterpret_cast<Vec2 *>(dst + 2 * i) = v;
}

template <typename Real>
int forest_forward(const ForestDims &d, bool fern, const Real *x, const Real *thr, const int64_t *ord, const Real *w,
                   Real *out, void *records, void *ws, size_t ws_bytes, hipStream_t stream, const ImageStore *image,
                   const FeatureNorm<Real> *norm_in) {
  if (is_empty(d)) return HT_OK;
  FeatureNorm<Real> norm;
  if (norm_in) norm = *norm_in;
  if (ws == nullptr || ws_bytes < forest_forward_workspace<Real>(d))
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: workspace too small for the forward pass.");
  ImageStore img{};
  if (image) img = *image;
  // the walk records' bound slots are cleared by whichever vertex-packing pre-pass runs below
  unsigned long long *slots = records ? records_bound_slots<Real>(d, records) : nullptr;
  if (img.nd && d.K == 1)
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: an image result needs inner data positions (inData of 3 or more dimensions).");
  // (the row kernels read the features as they lie in memory: a normalising call takes the tile kernels below)
  if (rows_ok<Real>(d) && norm.mean == nullptr) {
    int wpitch = weight_pitch<Real>(d);
    const bool shifted =
        odd_pairs_ok<Real>(d, wpitch, out) &&
        (reinterpret_cast<uintptr_t>(ws) + vertex_bytes<Real>(d)) % (2 * sizeof(Real)) == 0;  // the padded table
    if (wpitch != d.M) {
      Real *padded = reinterpret_cast<Real *>(static_cast<unsigned char *>(ws) + vertex_bytes<Real>(d));
      const long long rows = (long long)d.T * d.L;
      const long long pairs = rows * wpitch / 2;
      int log2_ppr = 0;
      while ((2 << log2_ppr) < wpitch) ++log2_ppr;
      if (d.M % 2 == 0 && (2 << log2_ppr) == wpitch && reinterpret_cast<uintptr_t>(w) % (2 * sizeof(Real)) == 0 &&
          (pairs + 255) / 256 <= 0x7fffffffLL) {
        hipLaunchKernelGGL(pad_rows_pairs_kernel<Real>, dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, stream, w,
                           padded, pairs, d.M, log2_ppr);
      } else {
        long long blocks = (rows * wpitch + 255) / 256;
        if (blocks > 16 * kNumCUs) blocks = 16 * kNumCUs;
        hipLaunchKernelGGL(pad_rows_kernel<Real>, dim3((unsigned)blocks), dim3(256), 0, stream, w, padded, rows, d.M,
                           wpitch, shifted, d.L);
      }
      HT_LAUNCH_CHECK("pad leaf rows");
      w = padded;
    }
    if constexpr (std::is_same<Real, float>::value) {
      if (quads_ok<Real>(d, fern)) {
        const int NQ = int(quads_per_tree(d.depth));
        const long long n = (long long)d.T * NQ;
        hipLaunchKernelGGL(pack_quads_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, thr, ord,
                           static_cast<QuadNode *>(ws), d.T, d.V, NQ, d.F, slots);
        HT_LAUNCH_CHECK("pack two-level vertices");
        return dispatch_rows<Real, false, true>(d, x, ws, w, wpitch, shifted, out, records, stream);
      }
    }
    int rc = pack_nodes<Real>(d, thr, ord, ws, stream, slots);
    if (rc != HT_OK) return rc;
    return fern ? dispatch_rows<Real, true, false>(d, x, ws, w, wpitch, shifted, out, records, stream)
                : dispatch_rows<Real, false, false>(d, x, ws, w, wpitch, shifted, out, records, stream);
  }
  int rc = pack_nodes<Real>(d, thr, ord, ws, stream, slots);
  if (rc != HT_OK) return rc;
  const Node<Real> *nodes = static_cast<const Node<Real> *>(ws);
  return fern ? dispatch_forward<Real, true>(d, x, nodes, w, out, records, stream, img, norm)
              : dispatch_forward<Real, false>(d, x, nodes, w, out, records, stream, img, norm);
}

// ---- maps on the row kernel's walk ----------------------------------------------------------------------------------
template <typename Real, bool FERN, bool QUAD, int BT>
static int launch_maps_rows(const ForestDims &d, const Real *x, const void *vertices, int64_t *leafmap, uint16_t *keys16,
                            Real *margins, int64_t *ordinals, hipStream_t stream) {
  constexpr int TPW = kWave / BT * kRowIlp;
  constexpr int TP = kForestThreads / kWave * TPW;
  const size_t lds = rows_lds_bytes<Real>(d.F, BT);
  const long long tiles = (d.S + BT - 1) / BT;
  int trees_per_block, gy;
  split_trees(tiles, d.T, TP, &trees_per_block, &gy);
  if (tiles > 0x7fffffffLL) return fail(HT_ERR_RUNTIME, "Error: too many sample tiles for one launch.");
  const int NQ = int(quads_per_tree(d.depth));
  if (leafmap || keys16) {
    auto kernel = maps_rows_kernel<Real, FERN, QUAD, BT, false>;
    HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));
    hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)gy), dim3(kForestThreads), lds, stream, d, x, vertices, NQ,
                       leafmap, keys16, (Real *)nullptr, (int64_t *)nullptr, trees_per_block);
    HT_LAUNCH_CHECK("forest maps (leaf keys)");
  }
  if (margins || ordinals) {
    auto kernel = maps_rows_kernel<Real, FERN, QUAD, BT, true>;
    HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));
    hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)gy), dim3(kForestThreads), lds, stream, d, x, vertices, NQ,
                       (int64_t *)nullptr, (uint16_t *)nullptr, margins, ordinals, trees_per_block);
    HT_LAUNCH_CHECK("forest maps (margins)");
  }
  return HT_OK;
}

template <typename Real, bool FERN, bool QUAD>
static int dispatch_maps_rows(const ForestDims &d, const Real *x, const void *vertices, int64_t *leafmap,
                              uint16_t *keys16, Real *margins, int64_t *ordinals, hipStream_t stream) {
  switch (pick_rows_tile<Real>(d.F)) {
    case 64: return launch_maps_rows<Real, FERN, QUAD, 64>(d, x, vertices, leafmap, keys16, margins, ordinals, stream);
    case 32: return launch_maps_rows<Real, FERN, QUAD, 32>(d, x, vertices, leafmap, keys16, margins, ordinals, stream);
    case 16: return launch_maps_rows<Real, FERN, QUAD, 16>(d, x, vertices, leafmap, keys16, margins, ordinals, stream);
    default: return launch_maps_rows<Real, FERN, QUAD, 8>(d, x, vertices, leafmap, keys16, margins, ordinals, stream);
  }
}

template <typename Real>
size_t forest_maps_rows_workspace(const ForestDims &d) {
  return rows_ok<Real>(d) ? vertex_bytes<Real>(d) : 0;
}

template <typename Real>
int forest_maps_rows(const ForestDims &d, bool fern, const Real *x, const Real *thr, const int64_t *ord,
                     int64_t *leafmap, uint16_t *keys16, Real *margins, int64_t *ordinals, void *ws,
                     hipStream_t stream) {
  if constexpr (std::is_same<Real, float>::value) {
    if (quads_ok<Real>(d, fern)) {
      const int NQ = int(quads_per_tree(d.depth));
      const long long n = (long long)d.T * NQ;
      hipLaunchKernelGGL(pack_quads_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, thr, ord,
                         static_cast<QuadNode *>(ws), d.T, d.V, NQ, d.F, (unsigned long long *)nullptr);
      HT_LAUNCH_CHECK("pack two-level vertices");
      return dispatch_maps_rows<Real, false, true>(d, x, ws, leafmap, keys16, margins, ordinals, stream);
    }
  }
  int rc = pack_nodes<Real>(d, thr, ord, ws, stream, nullptr);
  if (rc != HT_OK) return rc;
  return fern ? dispatch_maps_rows<Real, true, false>(d, x, ws, leafmap, keys16, margins, ordinals, stream)
              : dispatch_maps_rows<Real, false, false>(d, x, ws, leafmap, keys16, margins, ordinals, stream);
}

#define HT_INSTANTIATE(Real)                                                                                          \
  template size_t packed_nodes_bytes<Real>(const ForestDims &);                                                       \
  template int pack_nodes<Real>(const ForestDims &, const Real *, const int64_t *, void *, hipStream_t,                \
                                unsigned long long *);                                                                \
  template size_t forest_forward_workspace<Real>(const ForestDims &);                                                 \
  template int forest_forward<Real>(const ForestDims &, bool, const Real *, const Real *, const int64_t *,            \
                                    const Real *, Real *, void *, void *, size_t, hipStream_t, const ImageStore *,    \
                                    const FeatureNorm<Real> *);                                                       \
  template size_t forest_maps_rows_workspace<Real>(const ForestDims &);                                               \
  template int forest_maps_rows<Real>(const ForestDims &, bool, const Real *, const Real *, const int64_t *,          \
                                      int64_t *, uint16_t *, Real *, int64_t *, void *, hipStream_t);
HT_INSTANTIATE(float)
HT_INSTANTIATE(double)
#undef HT_INSTANTIATE

}  // namespace ht
