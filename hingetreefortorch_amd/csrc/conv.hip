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
constexpr int kConvIlp = 4;  // channels whose walks a thread of the tiled kernels interleaves (hides LDS latency)

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

// ---------------------------------------------------------------------------------------------------------------
// tiled kernels for 1 and 2 spatial dims
// ---------------------------------------------------------------------------------------------------------------
// A workgroup owns a TZ x TY x TX tile of output positions of one image (one thread per position; TZ = 1 for 1-d and
// 2-d data, TY = 1 as well for 1-d) and keeps the input region that tile reads -- all C channels, zeros where the region
// leaves the image -- in LDS. The trees of one out channel (C trees) are staged in LDS as (threshold, tile offset of the
// tap) pairs, so a walk step is two LDS reads and no address arithmetic beyond one add, and the padding needs no test.
// Every byte of x is read from memory once per tile instead of once per (out channel, vertex visit).
struct ConvTile {
  int D, H, W, OD, OH, OW;
  int kd, kh, kw, sz, sy, sx, pz, py, px, dz, dy, dx;
  int TZ, TY, TX, log2_tx, log2_ty;  // output tile, TZ * TY * TX == threads of the workgroup, powers of two
  int ID, IH, IW, PL, TSZ;           // input region of a tile: PL = IH * IW cells per slice, TSZ = ID * PL
  int tiles_z, tiles_y, tiles_x;
  int taps;
  __host__ __device__ long long tiles() const { return (long long)tiles_z * tiles_y * tiles_x; }
  __host__ __device__ long long positions() const { return (long long)OD * OH * OW; }
};

static bool make_tile(const ConvGeom &g, ConvTile *t, int threads = kConvThreads) {
  // the last dimension is x, the one before it y, the one before that z; missing ones have extent 1
  int size[3] = {1, 1, 1}, osz[3] = {1, 1, 1}, ker[3] = {1, 1, 1}, str[3] = {1, 1, 1}, pad[3] = {0, 0, 0},
      dil[3] = {1, 1, 1};
  for (int dd = 0; dd < g.nd; ++dd) {
    const int at = 3 - g.nd + dd;
    size[at] = g.size[dd], osz[at] = g.osz[dd], ker[at] = g.ker[dd];
    str[at] = g.str[dd], pad[at] = g.pad[dd], dil[at] = g.dil[dd];
  }
  t->D = size[0], t->H = size[1], t->W = size[2];
  t->OD = osz[0], t->OH = osz[1], t->OW = osz[2];
  t->kd = ker[0], t->kh = ker[1], t->kw = ker[2];
  t->sz = str[0], t->sy = str[1], t->sx = str[2];
  t->pz = pad[0], t->py = pad[1], t->px = pad[2];
  t->dz = dil[0], t->dy = dil[1], t->dx = dil[2];
  int tx = threads;  // widest power-of-two tile row that the output needs
  while (tx > 32 && tx / 2 >= t->OW) tx /= 2;
  if ((t->OH > 1 || t->OD > 1) && tx > 32) tx = 32;
  int ty = threads / tx;
  if (t->OD > 1) {
    // three dimensions: a brick rather than a slab, so that the input region (and the dX image flushed from it) is
    // a small multiple of the tile
    while (tx > 16 || (tx > 4 && tx / 2 >= t->OW)) tx /= 2;
    ty = 8;
    while (ty > 1 && ty / 2 >= t->OH) ty /= 2;
    if (threads / (tx * ty) > 8) ty = threads / (tx * 8);  // at most eight slices per brick
  }
  t->TX = tx;
  t->TY = ty;
  t->TZ = threads / (tx * ty);
  t->log2_tx = t->log2_ty = 0;
  while ((1 << t->log2_tx) < tx) ++t->log2_tx;
  while ((1 << t->log2_ty) < ty) ++t->log2_ty;
  t->ID = (t->TZ - 1) * t->sz + (t->kd - 1) * t->dz + 1;
  t->IH = (t->TY - 1) * t->sy + (t->kh - 1) * t->dy + 1;
  t->IW = (t->TX - 1) * t->sx + (t->kw - 1) * t->dx + 1;
  const long long tsz = (long long)t->ID * t->IH * t->IW;
  if (tsz > (1 << 20)) return false;
  t->PL = t->IH * t->IW;
  t->TSZ = int(tsz);
  t->tiles_z = (t->OD + t->TZ - 1) / t->TZ;
  t->tiles_y = (t->OH + t->TY - 1) / t->TY;
  t->tiles_x = (t->OW + t->TX - 1) / t->TX;
  t->taps = g.taps;
  return t->tiles() <= 0x7fffffffLL;
}

// Where a thread stands: its tile (index within the image), its output position, and the offset of that position's
// patch anchor inside the tile's input region.
struct ConvPos {
  int tzi, tyi, txi;  // tile
  int base;           // anchor offset in the region
  long long pos;      // output position within (image, out channel)
  bool live;          // the position exists
};

__device__ __forceinline__ ConvPos conv_pos(const ConvTile &g, unsigned tile_index, unsigned tid) {
  ConvPos p;
  const unsigned row = tile_index / unsigned(g.tiles_x);
  p.txi = int(tile_index - row * unsigned(g.tiles_x));
  p.tzi = int(row / unsigned(g.tiles_y));
  p.tyi = int(row - unsigned(p.tzi) * unsigned(g.tiles_y));
  const int tx = int(tid) & (g.TX - 1), ty = (int(tid) >> g.log2_tx) & (g.TY - 1),
            tz = int(tid) >> (g.log2_tx + g.log2_ty);
  const int oz = p.tzi * g.TZ + tz, oy = p.tyi * g.TY + ty, ox = p.txi * g.TX + tx;
  p.live = oz < g.OD && oy < g.OH && ox < g.OW;
  p.base = tz * g.sz * g.PL + ty * g.sy * g.IW + tx * g.sx;
  p.pos = ((long long)oz * g.OH + oy) * g.OW + ox;
  return p;
}

// Image coordinates of cell r of the tile's input region: the flat offset inside a channel image, or -1 outside.
__device__ __forceinline__ long long region_cell(const ConvTile &g, const ConvPos &p, int r) {
  const int iz = r / g.PL, r2 = r - iz * g.PL;
  const int iy = r2 / g.IW, ix = r2 - iy * g.IW;
  const int gz = p.tzi * g.TZ * g.sz - g.pz + iz, gy = p.tyi * g.TY * g.sy - g.py + iy,
            gx = p.txi * g.TX * g.sx - g.px + ix;
  if (gz < 0 || gz >= g.D || gy < 0 || gy >= g.H || gx < 0 || gx >= g.W) return -1;
  return ((long long)gz * g.H + gy) * g.W + gx;
}

// Magnitude bits of a float (its bit pattern without the sign orders like |v|, every NaN above infinity); 0 for doubles,
// whose callers do not use the bound.
__device__ __forceinline__ uint32_t magnitude_bits(float v) { return __float_as_uint(v) & 0x7fffffffu; }
__device__ __forceinline__ uint32_t magnitude_bits(double) { return 0u; }

// Largest value over the wavefront, to every lane (row operations of the vector ALU, then across the rows).
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  v = max(v, uint32_t(__builtin_amdgcn_update_dpp(0, int(v), 0xB1, 0xF, 0xF, true)));   // quad_perm [1,0,3,2]
  v = max(v, uint32_t(__builtin_amdgcn_update_dpp(0, int(v), 0x4E, 0xF, 0xF, true)));   // quad_perm [2,3,0,1]
  v = max(v, uint32_t(__builtin_amdgcn_update_dpp(0, int(v), 0x141, 0xF, 0xF, true)));  // row_half_mirror
  v = max(v, uint32_t(__builtin_amdgcn_update_dpp(0, int(v), 0x140, 0xF, 0xF, true)));  // row_mirror
  // every lane of a row of 16 now holds its row's maximum: the four rows meet in scalar registers
  const uint32_t r0 = uint32_t(__builtin_amdgcn_readlane(int(v), 0)), r1 = uint32_t(__builtin_amdgcn_readlane(int(v), 16));
  const uint32_t r2 = uint32_t(__builtin_amdgcn_readlane(int(v), 32)), r3 = uint32_t(__builtin_amdgcn_readlane(int(v), 48));
  return max(max(r0, r1), max(r2, r3));
}

// Cooperative load of the input region of tile `at` of image b, all channels: a thread owns one or two cells of
// the region and copies them channel by channel (the coordinate arithmetic is done once per cell, not per element).
// c0 / count: the window of channels to load (all of them by default); plane c0 + k goes to tile plane k.
// bound (optional): an LDS word that receives the largest magnitude_bits of the tile's values.
template <typename Real, bool CHECK = false>
__device__ __forceinline__ void load_conv_tile(Real *tile, const Real *__restrict__ x, const ConvTile &g, int C,
                                               long long b, const ConvPos &at, int *special, int c0 = 0,
                                               int count = -1, uint32_t *bound = nullptr) {
  const long long chan = (long long)g.D * g.H * g.W;
  const Real *img = x + (b * C + c0) * chan;
  if (count >= 0) C = count;
  uint32_t big = 0u;
  for (int e = threadIdx.x; e < g.TSZ; e += int(blockDim.x)) {
    const long long cell = region_cell(g, at, e);
    Real *q = tile + e;
    if (cell >= 0) {
      const Real *p = img + cell;
      bool plain = true;
#pragma unroll 4
      for (int c = 0; c < C; ++c) {
        const Real v = p[c * chan];
        if (CHECK) plain = plain && plain_feature(v);
        big = max(big, magnitude_bits(v));
        q[c * g.TSZ] = v;
      }
      if (CHECK && !plain) *special = 1;  // see walk_paths_plain; never reset, every writer stores the same value
    } else {
      for (int c = 0; c < C; ++c) q[c * g.TSZ] = Real(0);
    }
  }
  if (bound) {  // (one atomic per wavefront: same-address atomics are served one lane at a time)
    big = wave_max_u32(big);
    if ((threadIdx.x & 63) == 0 && big) atomicMax(bound, big);
  }
}

// The dX image of a tile's input region (fp64, C planes of TSZ cells) added to dx; cells outside the image are dropped
// like the reference drops padded taps. Regions of neighbouring tiles overlap, hence atomics.
// fixed: the cells are 64-bit integers, multiples of `unit` (see conv_tiled_backward_kernel).
template <typename Real>
__device__ __forceinline__ void flush_dx_image(const double *acc, const ConvTile &g, const ConvPos &at, int C,
                                               Real *dx_first /* image b, first channel of the window */,
                                               bool fixed = false, double unit = 1.0) {
  const long long chan = (long long)g.D * g.H * g.W;
  for (int i = threadIdx.x; i < C * g.TSZ; i += int(blockDim.x)) {
    const double v = fixed ? double(reinterpret_cast<const long long *>(acc)[i]) * unit : acc[i];
    if (v == 0.0) continue;
    const int c = i / g.TSZ, r = i - c * g.TSZ;
    const long long cell = region_cell(g, at, r);
    if (cell >= 0) atomicAdd(dx_first + c * chan + cell, Real(v));
  }
}

// Offset of every tap from the patch anchor inside the tile's input region; filled once per workgroup (a barrier
// separates it from the first staging of trees), so that staging a vertex is a table lookup instead of divisions.
__device__ __forceinline__ void fill_tap_offsets(int *tapoff, const ConvTile &g) {
  for (int tap = threadIdx.x; tap < g.taps; tap += int(blockDim.x)) {
    const int kz = tap / (g.kh * g.kw), rest = tap - kz * (g.kh * g.kw);
    const int ky = rest / g.kw, kx = rest - ky * g.kw;
    tapoff[tap] = kz * g.dz * g.PL + ky * g.dy * g.IW + kx * g.dx;
  }
}

// Trees (and optionally leaf weights) of out channel j into LDS.
// c0 / count: the window of channels whose trees are staged (all of them by default).
// thr_bound / w_bound (optional): LDS words that receive the largest magnitude_bits of the staged thresholds / weights.
template <typename Real, bool CHECK = false>
__device__ __forceinline__ void stage_conv_trees(Node<Real> *nodes, Real *wl, const ConvTile &g, const int *tapoff,
                                                 int C, int V, int LM, int j, const Real *__restrict__ thr,
                                                 const int64_t *__restrict__ ord, const Real *__restrict__ w,
                                                 int *special, int c0 = 0, int count = -1,
                                                 uint32_t *thr_bound = nullptr, uint32_t *w_bound = nullptr) {
  const long long tree0 = (long long)j * C + c0;
  if (count >= 0) C = count;
  const long long first = tree0 * V;
  uint32_t big = 0u;
  for (int i = threadIdx.x; i < C * V; i += int(blockDim.x)) {
    Node<Real> n;
    n.thr = thr[first + i];
    n.ord = tapoff[clamp_ordinal(ord[first + i], g.taps)];
    nodes[i] = n;
    big = max(big, magnitude_bits(n.thr));
    if (CHECK && !plain_threshold(n.thr)) *special = 1;
  }
  if (thr_bound) {  // (one atomic per wavefront: same-address atomics are served one lane at a time)
    big = wave_max_u32(big);
    if ((threadIdx.x & 63) == 0 && big) atomicMax(thr_bound, big);
  }
  if (wl) {
    const long long wfirst = tree0 * LM;
    big = 0u;
    for (int i = threadIdx.x; i < C * LM; i += int(blockDim.x)) {
      const Real v = w[wfirst + i];
      big = max(big, magnitude_bits(v));
      wl[i] = v;
    }
    if (w_bound) {
      big = wave_max_u32(big);
      if ((threadIdx.x & 63) == 0 && big) atomicMax(w_bound, big);
    }
  }
}

struct ConvLds {
  size_t tile, acc_x, nodes, wl, acc_w, acc_t, taps, flag, total;
};

template <typename Real>
static ConvLds conv_lds_layout(const ConvTile &t, int C, int V, int LM, bool dx_acc, bool tree_acc, bool w_lds) {
  ConvLds l{};
  size_t at = 0;
  l.tile = at;
  at += align_up(size_t(C) * t.TSZ * sizeof(Real), 16);
  l.acc_x = at;
  if (dx_acc) at += align_up(size_t(C) * t.TSZ * sizeof(double), 16);
  l.nodes = at;
  at += align_up(size_t(C) * V * sizeof(Node<Real>), 16);
  l.wl = at;
  if (w_lds) at += align_up(size_t(C) * LM * sizeof(Real), 16);
  l.acc_w = at;
  if (tree_acc) at += align_up(size_t(C) * LM * sizeof(double), 16);
  l.acc_t = at;
  if (tree_acc) at += align_up(size_t(C) * V * sizeof(double), 16);
  l.taps = at;  // tap -> offset in the tile's input region
  at += align_up(size_t(t.taps) * sizeof(int), 16);
  // word 0: set once the tile or the staged trees hold a value that rules out walk_paths_plain; words 1 .. 7: the
  // magnitude bounds behind the fixed-point cells of conv_tiled_backward_kernel
  l.flag = at;
  at += 64;
  l.total = at;
  return l;
}

// kConvIlp walks of one output position through the staged trees nd[] over the tile planes px[]: the short form where
// the workgroup's data allow it (see walk_paths_plain), else the general one.
template <typename Real, bool FERN, bool TRACK>
__device__ __forceinline__ void conv_walks(bool plain, int depth, const Node<Real> *const (&nd)[kConvIlp],
                                           const Real *const (&px)[kConvIlp], WalkResult<Real> (&r)[kConvIlp]) {
  if constexpr (std::is_same<Real, float>::value) {
    if (plain) {
      const Node<float> *nd1[kConvIlp];  // trees: addressed by the 1-based heap index
#pragma unroll
      for (int i = 0; i < kConvIlp; ++i) nd1[i] = nd[i] - (FERN ? 0 : 1);
      if constexpr (TRACK) {
        TrackedPath st[kConvIlp];
        walk_paths_plain_tracked<FERN, kConvIlp>(
            depth, [&](int i, uint32_t at) { return nd1[i][at]; }, [&](int i, int off) { return px[i][off]; }, st);
#pragma unroll
        for (int i = 0; i < kConvIlp; ++i) {
          r[i].key = st[i].key(depth);
          r[i].vertex = st[i].template vertex<FERN>(depth);
          r[i].ord = st[i].ordinal();
          r[i].margin = 0.f - st[i].t;  // x - thr, exactly; +0.0 where they are equal
        }
      } else {
        walk_paths_plain<FERN, kConvIlp>(
            depth, [&](int i, uint32_t at) { return nd1[i][at]; }, [&](int i, int off) { return px[i][off]; }, r);
      }
      return;
    }
  }
  walk_paths<Real, FERN, TRACK, kConvIlp>(
      depth, [&](int i, uint32_t at) { return nd[i][at]; }, [&](int i, int off) { return px[i][off]; }, r);
}

// MREG = outputs per leaf kept in registers per pass over the channels (1, 4 or 16: the smallest that holds M, so the
// common single-output case carries no per-output loop at all).
// Channel windows: where the tile planes and the staged trees of all C channels would leave room for one workgroup per
// CU only (many channels, deep trees, many outputs per leaf), the workgroup takes c_per channels at a time -- loads
// their planes, then for every out channel stages their trees and adds their terms to what the earlier windows left
// in `out`. The terms of a position are still added one by one in ascending channel order to the same running value
// (it merely passes through memory between windows), so the result is bit for bit the one of a single pass.
template <typename Real, bool FERN, int MREG>
__global__ __launch_bounds__(kConvThreads) void conv_tiled_forward_kernel(ConvTile g, ConvLds lay, int C_all, int c_per,
                                                                          int Cout, int depth, int V, int L, int M,
                                                                          int j_per, const Real *__restrict__ x,
                                                                          const Real *__restrict__ thr,
                                                                          const int64_t *__restrict__ ord,
                                                                          const Real *__restrict__ w,
                                                                          Real *__restrict__ out) {
  extern __shared__ __align__(16) unsigned char smem[];
  Real *tile = reinterpret_cast<Real *>(smem + lay.tile);
  Node<Real> *nodes = reinterpret_cast<Node<Real> *>(smem + lay.nodes);
  Real *wl = reinterpret_cast<Real *>(smem + lay.wl);
  const ConvPos at = conv_pos(g, blockIdx.x, threadIdx.x);
  const long long b = blockIdx.z;
  int *special = reinterpret_cast<int *>(smem + lay.flag);
  int *tapoff = reinterpret_cast<int *>(smem + lay.taps);
  fill_tap_offsets(tapoff, g);
  if (threadIdx.x == 0) *special = 0;
  const bool live = at.live;
  const Real *mine = tile + at.base;
  const int LM = L * M;
  const int j_begin = blockIdx.y * j_per, j_end = min(Cout, j_begin + j_per);
  for (int c0 = 0; c0 < C_all; c0 += c_per) {
    const int C = min(c_per, C_all - c0);
    __syncthreads();  // the flag is cleared / the previous window's planes and trees are no longer read
    load_conv_tile<Real, true>(tile, x, g, C_all, b, at, special, c0, C);
    for (int j = j_begin; j < j_end; ++j) {
      __syncthreads();  // the planes are complete / the previous out channel's trees are no longer read
      stage_conv_trees<Real, true>(nodes, wl, g, tapoff, C_all, V, LM, j, thr, ord, w, special, c0, C);
      __syncthreads();
      if (!live) continue;
      const bool plain = *special == 0;
      Real *o = out + ((b * Cout + j) * g.positions() + at.pos) * M;
      for (int m0 = 0; m0 < M; m0 += MREG) {
        const int mc = min(MREG, M - m0);
        Real acc[MREG];
#pragma unroll
        for (int m = 0; m < MREG; ++m) acc[m] = (c0 == 0 || (MREG != 1 && m >= mc)) ? Real(0) : o[m0 + m];
        for (int c = 0; c < C; c += kConvIlp) {
          // several channels' walks interleaved; their terms are still added in ascending channel order
          WalkResult<Real> r[kConvIlp];
          const Node<Real> *nd[kConvIlp];
          const Real *px[kConvIlp];
#pragma unroll
          for (int i = 0; i < kConvIlp; ++i) {
            const int ci = min(c + i, C - 1);  // surplus slots re-walk the last channel, unused
            nd[i] = nodes + ci * V;
            px[i] = mine + ci * g.TSZ;
          }
          conv_walks<Real, FERN, false>(plain, depth, nd, px, r);
#pragma unroll
          for (int i = 0; i < kConvIlp; ++i) {
            if (c + i >= C) break;
            const Real a = r[i].margin;  // |margin|
            const Real *row = wl + ((c + i) * L + r[i].key) * M + m0;
#pragma unroll
            for (int m = 0; m < MREG; ++m)
              if (MREG == 1 || m < mc) acc[m] = acc[m] + row[m] * a;
          }
        }
#pragma unroll
        for (int m = 0; m < MREG; ++m)
          if (MREG == 1 || m < mc) o[m0 + m] = acc[m];
      }
    }
  }
}

// dX: tile-stationary over all out channels; c = sign(margin) * sum_m w * g goes into an fp64 LDS image of the tile's
// input region (fp64 because that is the fast LDS floating-point atomic on gfx950), flushed once with global atomics
// (regions of neighbouring tiles overlap). Cells outside the image are dropped like the reference drops padded taps.
template <typename Real, bool FERN>
__global__ __launch_bounds__(kConvThreads) void conv_tiled_dx_kernel(ConvTile g, ConvLds lay, int C, int Cout,
                                                                     int depth, int V, int L, int M, int j_per,
                                                                     const Real *__restrict__ x,
                                                                     const Real *__restrict__ thr,
                                                                     const int64_t *__restrict__ ord,
                                                                     const Real *__restrict__ w,
                                                                     const Real *__restrict__ gout, Real *dx) {
  extern __shared__ __align__(16) unsigned char smem[];
  Real *tile = reinterpret_cast<Real *>(smem + lay.tile);
  double *acc = reinterpret_cast<double *>(smem + lay.acc_x);
  Node<Real> *nodes = reinterpret_cast<Node<Real> *>(smem + lay.nodes);
  Real *wl = reinterpret_cast<Real *>(smem + lay.wl);
  const ConvPos at = conv_pos(g, blockIdx.x, threadIdx.x);
  const long long b = blockIdx.z;
  int *special = reinterpret_cast<int *>(smem + lay.flag);
  int *tapoff = reinterpret_cast<int *>(smem + lay.taps);
  fill_tap_offsets(tapoff, g);
  if (threadIdx.x == 0) *special = 0;
  __syncthreads();
  load_conv_tile<Real, true>(tile, x, g, C, b, at, special);
  for (int i = threadIdx.x; i < C * g.TSZ; i += kConvThreads) acc[i] = 0.0;
  const bool live = at.live;
  const int base = at.base;
  const Real *mine = tile + base;
  const int LM = L * M;
  const int j_begin = blockIdx.y * j_per, j_end = min(Cout, j_begin + j_per);
  for (int j = j_begin; j < j_end; ++j) {
    __syncthreads();
    stage_conv_trees<Real, true>(nodes, wl, g, tapoff, C, V, LM, j, thr, ord, w, special);
    __syncthreads();
    if (!live) continue;
    const bool plain = *special == 0;
    const Real *gp = gout + ((b * Cout + j) * g.positions() + at.pos) * M;
    for (int c = 0; c < C; c += kConvIlp) {
      WalkResult<Real> r[kConvIlp];
      const Node<Real> *nd[kConvIlp];
      const Real *px[kConvIlp];
#pragma unroll
      for (int i = 0; i < kConvIlp; ++i) {
        const int ci = min(c + i, C - 1);
        nd[i] = nodes + ci * V;
        px[i] = mine + ci * g.TSZ;
      }
      conv_walks<Real, FERN, true>(plain, depth, nd, px, r);
#pragma unroll
      for (int i = 0; i < kConvIlp; ++i) {
        if (c + i >= C) break;
        const Real *row = wl + ((c + i) * L + r[i].key) * M;
        Real cs = Real(0);
        for (int m = 0; m < M; ++m) cs += row[m] * gp[m];
        cs = ht_sign(r[i].margin) * cs;
        atomicAdd(acc + (c + i) * g.TSZ + base + int(r[i].ord), double(cs));  // r.ord is the tap's tile offset
      }
    }
  }
  __syncthreads();
  flush_dx_image(acc, g, at, C, dx + b * C * (long long)g.D * g.H * g.W);
}

// dThr and dW: a workgroup owns out channel blockIdx.x and visits every blockIdx.y-th (image, tile); the gradients of
// its C trees are accumulated in fp64 LDS tables over all of those visits and flushed once.
template <typename Real, bool FERN>
__global__ __launch_bounds__(kConvThreads) void conv_tiled_trees_kernel(ConvTile g, ConvLds lay, int C, int Cout,
                                                                        int depth, int V, int L, int M, long long items,
                                                                        const Real *__restrict__ x,
                                                                        const Real *__restrict__ thr,
                                                                        const int64_t *__restrict__ ord,
                                                                        const Real *__restrict__ w,
                                                                        const Real *__restrict__ gout, Real *dthr,
                                                                        Real *dw) {
  extern __shared__ __align__(16) unsigned char smem[];
  Real *tile = reinterpret_cast<Real *>(smem + lay.tile);
  Node<Real> *nodes = reinterpret_cast<Node<Real> *>(smem + lay.nodes);
  Real *wl = reinterpret_cast<Real *>(smem + lay.wl);
  double *acc_w = reinterpret_cast<double *>(smem + lay.acc_w);
  double *acc_t = reinterpret_cast<double *>(smem + lay.acc_t);
  const int j = blockIdx.x;
  const int LM = L * M;
  int *special = reinterpret_cast<int *>(smem + lay.flag);
  int *tapoff = reinterpret_cast<int *>(smem + lay.taps);
  fill_tap_offsets(tapoff, g);
  if (threadIdx.x == 0) *special = 0;
  __syncthreads();
  stage_conv_trees<Real, true>(nodes, wl, g, tapoff, C, V, LM, j, thr, ord, w, special);
  for (int i = threadIdx.x; i < C * LM; i += kConvThreads) acc_w[i] = 0.0;
  for (int i = threadIdx.x; i < C * V; i += kConvThreads) acc_t[i] = 0.0;
  const long long tiles = g.tiles();
  const int skew = int(threadIdx.x & 63u) % C;
  for (long long it = blockIdx.y; it < items; it += gridDim.y) {
    const long long b = it / tiles;
    const ConvPos at = conv_pos(g, unsigned(it - b * tiles), threadIdx.x);
    const Real *mine = tile + at.base;
    __syncthreads();  // the previous tile is no longer read (first pass: the staged trees are complete)
    load_conv_tile<Real, true>(tile, x, g, C, b, at, special);
    __syncthreads();
    const bool plain = *special == 0;
    if (!at.live) continue;
    const Real *gp = gout + ((b * Cout + j) * g.positions() + at.pos) * M;
    for (int c = 0; c < C; c += kConvIlp) {
      WalkResult<Real> r[kConvIlp];
      const Node<Real> *nd[kConvIlp];
      const Real *px[kConvIlp];
      int ch[kConvIlp];
#pragma unroll
      for (int i = 0; i < kConvIlp; ++i) {
        // Lane l takes the channels in the order skew(l), skew(l) + 1, ... (mod C): at any moment the lanes of a
        // wavefront are spread over min(C, 64) trees, so the root-heavy threshold table sees that many times fewer
        // same-address atomics than with all lanes on one tree.
        int ci = min(c + i, C - 1) + skew;
        ci = ci >= C ? ci - C : ci;
        ch[i] = ci;
        nd[i] = nodes + ci * V;
        px[i] = mine + ci * g.TSZ;
      }
      conv_walks<Real, FERN, true>(plain, depth, nd, px, r);
#pragma unroll
      for (int i = 0; i < kConvIlp; ++i) {
        if (c + i >= C) break;
        const Real a = ht_abs(r[i].margin);
        const int cell = (ch[i] * L + int(r[i].key)) * M;
        Real cs = Real(0);
        for (int m = 0; m < M; ++m) {
          const Real gv = gp[m];
          cs += wl[cell + m] * gv;
          if (dw) atomicAdd(acc_w + cell + m, double(a * gv));
        }
        if (dthr) atomicAdd(acc_t + ch[i] * V + int(r[i].vertex), -double(ht_sign(r[i].margin) * cs));
      }
    }
  }
  __syncthreads();
  if (dw)
    for (int i = threadIdx.x; i < C * LM; i += kConvThreads)
      if (acc_w[i] != 0.0) atomicAdd(dw + (long long)j * C * LM + i, Real(acc_w[i]));
  if (dthr)
    for (int i = threadIdx.x; i < C * V; i += kConvThreads)
      if (acc_t[i] != 0.0) atomicAdd(dthr + (long long)j * C * V + i, Real(acc_t[i]));
}

// All three gradients from ONE walk per (position, out channel, channel), for callers that want dX together with dThr
// or dW: tile-stationary like the dX kernel, with the fp64 tables of the current out channel's trees beside the dX
// image. A workgroup serves a window of c_per channels (its tile planes, dX image and trees): with all 16 channels of
// the benchmark shape one workgroup fills the LDS and a SIMD holds two wavefronts, with 8 it holds four, which hides
// the chains of dependent LDS reads that a walk is (2.74 -> 2.47 ms). The tree tables are flushed to memory with atomics after each out channel (C * (V + L * M) cells per NT
// positions x C walks), which is what the second walk of the two-kernel form is traded for; workgroups start at
// different out channels so that those atomics spread over all trees' addresses. NT = 512: the larger tile halves the
// flushes and the tree staging per walk, and one workgroup fills a CU's wavefront slots the way two smaller ones do.
// M1: one output per leaf, known at compile time (no loop over outputs; the position's upstream gradient is loaded once
// per out channel instead of once per walk).
template <typename Real, bool FERN, int NT, bool M1>
__global__ __launch_bounds__(NT) void conv_tiled_backward_kernel(ConvTile g, ConvLds lay, int C_all, int c_per, int Cout,
                                                                 int depth, int V, int L, int M, int j_per,
                                                                 const Real *__restrict__ x,
                                                                 const Real *__restrict__ thr,
                                                                 const int64_t *__restrict__ ord,
                                                                 const Real *__restrict__ w,
                                                                 const Real *__restrict__ gout, Real *dx, Real *dthr,
                                                                 Real *dw) {
  extern __shared__ __align__(16) unsigned char smem[];
  Real *tile = reinterpret_cast<Real *>(smem + lay.tile);
  double *acc = reinterpret_cast<double *>(smem + lay.acc_x);
  Node<Real> *nodes = reinterpret_cast<Node<Real> *>(smem + lay.nodes);
  Real *wl = reinterpret_cast<Real *>(smem + lay.wl);
  double *acc_w = reinterpret_cast<double *>(smem + lay.acc_w);
  double *acc_t = reinterpret_cast<double *>(smem + lay.acc_t);
  const ConvPos at = conv_pos(g, blockIdx.x, threadIdx.x);
  const long long b = blockIdx.z;
  // blockIdx.y = (block of out channels, window of channels): a workgroup holds the tile planes, the dX image and the
  // trees of c_per channels only, so that several workgroups fit a CU
  const int c_blocks = (C_all + c_per - 1) / c_per;
  const int c0 = int(blockIdx.y % unsigned(c_blocks)) * c_per, j_block = int(blockIdx.y / unsigned(c_blocks));
  const int C = min(c_per, C_all - c0);
  int *special = reinterpret_cast<int *>(smem + lay.flag);
  int *tapoff = reinterpret_cast<int *>(smem + lay.taps);
  fill_tap_offsets(tapoff, g);
  const int LM = L * M;
  // single-output float trees walk by the sign bit where the data allow it (walk_paths_plain_tracked)
  constexpr bool kLeanWalk = M1 && std::is_same<Real, float>::value;
  // Float data: the LDS cells are 64-bit integers. ds_add_u64 costs 13 cycles per wave instruction where ds_add_f64
  // costs 23, and the three atomics of a walk are most of what this kernel does with its LDS (backward of 32 images
  // [16,128,128] -> 64 channels, depth 6: 2.47 -> 2.0 ms). A term is scaled by a power of two that puts the largest
  // possible one just below 2^29, rounded to an integer once, and added; the workgroup finds the bounds behind the
  // scales in the data it stages anyway: max|x| of its tile, and per out channel max|g| of its positions, max|thr| and
  // max|w| of the staged trees (magnitude bits into LDS words 1 .. 7 of the flag area). dW terms are |thr - x| * g,
  // dThr and dX terms sign * sum_m w * g. The per-out-channel tables are flushed per out channel with that channel's
  // unit; the dX image lives through all of them, so it is shifted right when a later out channel needs a coarser
  // unit. A bound that is not finite (or scales beyond float's exponent range) puts the out channel -- for the dX image:
  // the rest of the workgroup's life -- on fp64 cells instead. Sums of at most a few thousand terms below 2^29 are
  // far from the ends of 64 bits.
  constexpr bool kFix = std::is_same<Real, float>::value;
  uint32_t *bnd = reinterpret_cast<uint32_t *>(smem + lay.flag);  // [1] tile; [2..4], [5..7]: g, thr, w of out channel parity 0, 1
  if (kLeanWalk || kFix) {
    if (threadIdx.x == 0) *special = 0;
    if (threadIdx.x >= 1 && threadIdx.x < 8) bnd[threadIdx.x] = 0u;
    __syncthreads();
  }
  load_conv_tile<Real, kLeanWalk>(tile, x, g, C_all, b, at, special, c0, C, kFix ? bnd + 1 : nullptr);
  for (int i = threadIdx.x; i < C * g.TSZ; i += NT) acc[i] = 0.0;
  for (int i = threadIdx.x; i < C * LM; i += NT) acc_w[i] = 0.0;
  for (int i = threadIdx.x; i < C * V; i += NT) acc_t[i] = 0.0;
  const bool live = at.live;
  const int base = at.base;
  const Real *mine = tile + base;
  // Lane l takes the channels in the order skew(l), skew(l) + 1, ... (mod C): the lanes of a wavefront are spread over
  // min(C, 64) trees' tables and dX planes, so the atomics of one instruction rarely meet on one address.
  const int lane = int(threadIdx.x & 63u);
  const int skew = ((lane & 31) + (lane >> 5) * (C >> 1)) % C;
  const int j_begin = j_block * j_per, j_count = min(Cout, j_begin + j_per) - j_begin;
  const int rot = int((blockIdx.x * 7u + blockIdx.z * 13u) % unsigned(j_count));
  // Fixed-point state (all of it wave uniform: every thread derives it from the same LDS words).
  // tab_fixed / unit_w / unit_c: cells and units of the tables of the out channel in hand; img_*: of the dX image.
  bool tab_fixed = false, img_fixed = kFix;
  int img_exp = -100000;  // exponent of the dX image's bound so far: its unit is 2^(img_exp - 29)
  float scale_w = 1.f, scale_t = 1.f, scale_x = 1.f;
  double unit_w = 1.0, unit_t = 1.0;
  // a term into a cell that holds either a double or, times `scale`, a 64-bit integer
  auto add = [&](double *cell, Real v, bool fixed, float scale) {
    if constexpr (kFix) {
      if (fixed) {
        atomicAdd(reinterpret_cast<unsigned long long *>(cell), (unsigned long long)(long long)__float2int_rn(v * scale));
        return;
      }
    }
    atomicAdd(cell, double(v));
  };
  // 2^e as a float, e inside the range of normal floats
  auto pow2f = [](int e) -> float { return __uint_as_float(uint32_t(e + 127) << 23); };
  auto g_of = [&](int jj) -> const Real * {
    const int j = j_begin + (jj + rot >= j_count ? jj + rot - j_count : jj + rot);
    return gout + ((b * Cout + j) * g.positions() + (live ? at.pos : 0)) * M;
  };
  auto j_of = [&](int jj) { return j_begin + (jj + rot >= j_count ? jj + rot - j_count : jj + rot); };
  // (single output) a position's gradient for the next out channel is requested while the current one is walked: its
  // bound is wanted before the barrier, where a fresh load's latency would be on every workgroup's critical path
  Real g_ahead = (M1 && live) ? *g_of(0) : Real(0);
  for (int jj = 0; jj < j_count; ++jj) {
    const int j = j_of(jj);
    uint32_t *now = bnd + 2 + 3 * (jj & 1), *next = bnd + 2 + 3 * ((jj & 1) ^ 1);
    __syncthreads();  // the tile and the zeroed tables are complete / the previous out channel's walks are done
    if (kFix && threadIdx.x < 3) next[threadIdx.x] = 0u;  // (read last before the barrier above)
    if (jj > 0) {
      // flush the previous out channel's tables (its trees are still known by index only: jp)
      const int jp = j_of(jj - 1);
      if (dw)
        for (int i = threadIdx.x; i < C * LM; i += NT) {
          const double v = tab_fixed ? double(reinterpret_cast<long long *>(acc_w)[i]) * unit_w : acc_w[i];
          if (v != 0.0) {
            atomicAdd(dw + ((long long)jp * C_all + c0) * LM + i, Real(v));
            acc_w[i] = 0.0;
          }
        }
      if (dthr)
        for (int i = threadIdx.x; i < C * V; i += NT) {
          const double v = tab_fixed ? double(reinterpret_cast<long long *>(acc_t)[i]) * unit_t : acc_t[i];
          if (v != 0.0) {
            atomicAdd(dthr + ((long long)jp * C_all + c0) * V + i, Real(v));
            acc_t[i] = 0.0;
          }
        }
    }
    stage_conv_trees<Real, kLeanWalk>(nodes, wl, g, tapoff, C_all, V, LM, j, thr, ord, w, special, c0, C,
                                      kFix ? now + 1 : nullptr, kFix ? now + 2 : nullptr);
    const Real *gp = gout + ((b * Cout + j) * g.positions() + (live ? at.pos : 0)) * M;
    const Real g_one = M1 ? g_ahead : Real(0);
    if constexpr (kFix) {
      // this position's largest |g|, over the wavefront, into the out channel's word
      uint32_t gb = 0u;
      if (live) {
        if (M1) {
          gb = magnitude_bits(g_one);
        } else {
          for (int m = 0; m < M; ++m) gb = max(gb, magnitude_bits(gp[m]));
        }
      }
      gb = wave_max_u32(gb);
      if ((threadIdx.x & 63) == 0 && gb) atomicMax(now, gb);
    }
    if (M1 && live && jj + 1 < j_count) g_ahead = *g_of(jj + 1);
    __syncthreads();
    if constexpr (kFix) {
      // bounds -> units. A float's exponent field e means |v| < 2^(e - 126).
      const uint32_t xb = bnd[1], gb = now[0], tb = now[1], wb = now[2];
      const bool finite = max(max(xb, gb), max(tb, wb)) < 0x7f800000u;
      const float g_max = __uint_as_float(gb);
      const float bound_w = (__uint_as_float(tb) + __uint_as_float(xb)) * g_max;
      const float bound_c = float(M) * __uint_as_float(wb) * g_max;
      const int exp_w = int(__float_as_uint(bound_w) >> 23) - 126, exp_c = int(__float_as_uint(bound_c) >> 23) - 126;
      // (a bound of zero: every term is zero, any unit will do)
      const bool ok_w = bound_w == 0.f || (exp_w > -90 && exp_w < 90), ok_c = bound_c == 0.f || (exp_c > -90 && exp_c < 90);
      tab_fixed = finite && ok_w && ok_c;
      if (tab_fixed) {
        const int ew = bound_w == 0.f ? 0 : exp_w, ec = bound_c == 0.f ? 0 : exp_c;
        scale_w = pow2f(29 - ew), unit_w = double(pow2f(ew - 29));
        scale_t = pow2f(29 - ec), unit_t = double(pow2f(ec - 29));
      }
      if (img_fixed) {
        const int ec = bound_c == 0.f ? -100000 : exp_c;
        if (!tab_fixed) {
          // the image goes over to fp64 cells for good
          if (img_exp > -100000) {
            const double unit = double(pow2f(img_exp - 29));
            for (int i = threadIdx.x; i < C * g.TSZ; i += NT) acc[i] = double(reinterpret_cast<long long *>(acc)[i]) * unit;
          }
          img_fixed = false;
          __syncthreads();
        } else if (ec > img_exp) {
          // a coarser unit from here on: what the image holds is shifted down to it
          if (img_exp > -100000) {
            const int shift = min(ec - img_exp, 63);
            for (int i = threadIdx.x; i < C * g.TSZ; i += NT)
              reinterpret_cast<long long *>(acc)[i] = reinterpret_cast<long long *>(acc)[i] >> shift;
            __syncthreads();
          }
          img_exp = ec;
        }
        if (img_fixed && img_exp > -100000) scale_x = pow2f(29 - img_exp);
      }
    }
    auto walks = [&]() {
    if (!live) return;
    if constexpr (kLeanWalk) {
      if (*special == 0) {
        // (the usual case, every cell an integer, as code of its own: no test per atomic)
        auto lean_walks = [&](auto all_fixed_tag) {
        constexpr bool ALL = decltype(all_fixed_tag)::value;
        const bool tab_f = ALL || tab_fixed, img_f = ALL || img_fixed;
        for (int c = 0; c < C; c += kConvIlp) {
          TrackedPath st[kConvIlp];
          const Node<float> *nd[kConvIlp];
          const float *px[kConvIlp];
          int ch[kConvIlp];
#pragma unroll
          for (int i = 0; i < kConvIlp; ++i) {
            int ci = min(c + i, C - 1) + skew;
            ci = ci >= C ? ci - C : ci;
            ch[i] = ci;
            nd[i] = nodes + ci * V - (FERN ? 0 : 1);  // trees: addressed by the 1-based heap index
            px[i] = mine + ci * g.TSZ;
          }
          walk_paths_plain_tracked<FERN, kConvIlp>(
              depth, [&](int i, uint32_t at) { return nd[i][at]; }, [&](int i, int off) { return px[i][off]; }, st);
#pragma unroll
          for (int i = 0; i < kConvIlp; ++i) {
            if (c + i >= C) break;
            const float t = st[i].t;  // thr - x at the selected vertex: margin = -t
            const int cell = ch[i] * L + int(st[i].key(depth));
            if (dw) add(acc_w + cell, ht_abs(t) * g_one, tab_f, scale_w);
            // sign(margin) * (w * g): the product with the sign bit of t flipped in, zero where the margin is zero
            const float wg = wl[cell] * g_one;
            const float cs = t == 0.f ? 0.f
                                      : __uint_as_float(__float_as_uint(wg) ^ (~__float_as_uint(t) & 0x80000000u));
            if (dthr) add(acc_t + ch[i] * V + int(st[i].template vertex<FERN>(depth)), -cs, tab_f, scale_t);
            add(acc + (px[i] - tile) + int(st[i].ordinal()), cs, img_f, scale_x);
          }
        }
        };
        if (tab_fixed && img_fixed)
          lean_walks(std::true_type{});
        else
          lean_walks(std::false_type{});
        return;
      }
    }
    for (int c = 0; c < C; c += kConvIlp) {
      WalkResult<Real> r[kConvIlp];
      const Node<Real> *nd[kConvIlp];
      const Real *px[kConvIlp];
      int ch[kConvIlp];
#pragma unroll
      for (int i = 0; i < kConvIlp; ++i) {
        int ci = min(c + i, C - 1) + skew;
        ci = ci >= C ? ci - C : ci;
        ch[i] = ci;
        nd[i] = nodes + ci * V;
        px[i] = mine + ci * g.TSZ;
      }
      conv_walks<Real, FERN, true>(false, depth, nd, px, r);
#pragma unroll
      for (int i = 0; i < kConvIlp; ++i) {
        if (c + i >= C) break;
        const Real a = ht_abs(r[i].margin);
        const int cell = (ch[i] * L + int(r[i].key)) * (M1 ? 1 : M);
        Real cs = Real(0);
        if (M1) {
          cs += wl[cell] * g_one;
          if (dw) add(acc_w + cell, a * g_one, tab_fixed, scale_w);
        } else {
          for (int m = 0; m < M; ++m) {
            const Real gv = gp[m];
            cs += wl[cell + m] * gv;
            if (dw) add(acc_w + cell + m, a * gv, tab_fixed, scale_w);
          }
        }
        cs = ht_sign(r[i].margin) * cs;
        if (dthr) add(acc_t + ch[i] * V + int(r[i].vertex), -cs, tab_fixed, scale_t);
        add(acc + ch[i] * g.TSZ + base + int(r[i].ord), cs, img_fixed, scale_x);  // r.ord is the tap's tile offset
      }
    }
    };
    walks();
  }
  __syncthreads();
  {
    const int jp = j_of(j_count - 1);
    if (dw)
      for (int i = threadIdx.x; i < C * LM; i += NT) {
        const double v = tab_fixed ? double(reinterpret_cast<long long *>(acc_w)[i]) * unit_w : acc_w[i];
        if (v != 0.0) atomicAdd(dw + ((long long)jp * C_all + c0) * LM + i, Real(v));
      }
    if (dthr)
      for (int i = threadIdx.x; i < C * V; i += NT) {
        const double v = tab_fixed ? double(reinterpret_cast<long long *>(acc_t)[i]) * unit_t : acc_t[i];
        if (v != 0.0) atomicAdd(dthr + ((long long)jp * C_all + c0) * V + i, Real(v));
      }
  }
  const bool img_ints = img_fixed && img_exp > -100000;
  flush_dx_image(acc, g, at, C, dx + (b * C_all + c0) * (long long)g.D * g.H * g.W, img_ints,
                 img_ints ? double(pow2f(img_exp - 29)) : 1.0);
}

constexpr int kConvWideThreads = 512;  // workgroup of the one-walk backward kernel

constexpr size_t kConvTiledLdsMax = 160 * 1024;  // LDS of a CU

// Out channels per workgroup of the tile-stationary kernels: all of them unless that leaves the device underfilled.
static int conv_j_per(long long tiles_total, int Cout) {
  long long want = tiles_total >= 4 * kNumCUs ? 1 : (4 * kNumCUs + tiles_total - 1) / (tiles_total > 0 ? tiles_total : 1);
  if (want > Cout) want = Cout;
  return int((Cout + want - 1) / want);
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
  ConvTile t;
  if (make_tile(g, &t)) {
    const int LM = L * int(s.M);
    // channels per window: all of them while four workgroups still fit a CU, else halved (not below four channels:
    // every window re-stages its trees per out channel and passes the running sums through memory). Trees of more
    // than 255 vertices are not split into windows: staging them costs more than a tile of positions gets out of
    // them, and where they do not fit at once the kernel below, which reads vertices through the caches, is faster.
    int c_per = int(s.C);
    ConvLds lay = conv_lds_layout<Real>(t, c_per, V, LM, false, false, true);
    while (V <= 255 && lay.total > kConvTiledLdsMax / 4 && c_per >= 8) {
      c_per = (c_per + 1) / 2;
      lay = conv_lds_layout<Real>(t, c_per, V, LM, false, false, true);
    }
    if (lay.total <= kConvTiledLdsMax) {
      const long long tiles = t.tiles();
      const int j_per = conv_j_per(tiles * s.B, int(s.Cout));
      const dim3 tgrid((unsigned)tiles, (unsigned)((s.Cout + j_per - 1) / j_per), (unsigned)s.B);
      auto kernel = fern ? conv_tiled_forward_kernel<Real, true, 16> : conv_tiled_forward_kernel<Real, false, 16>;
      if (s.M == 1) kernel = fern ? conv_tiled_forward_kernel<Real, true, 1> : conv_tiled_forward_kernel<Real, false, 1>;
      else if (s.M <= 4) kernel = fern ? conv_tiled_forward_kernel<Real, true, 4> : conv_tiled_forward_kernel<Real, false, 4>;
      HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));
      hipLaunchKernelGGL(kernel, tgrid, dim3(kConvThreads), lay.total, stream, t, lay, int(s.C), c_per, int(s.Cout),
                         int(s.depth), V, L, int(s.M), j_per, x, thr, ord, w, out);
      HT_LAUNCH_CHECK("conv forward (tiled)");
      return HT_OK;
    }
  }
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
  HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));
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
  ConvTile t;
  // dX together with a tree gradient: one walk serves all of them where the tables fit beside the dX image, with the
  // wide workgroup first and the ordinary one for shapes whose wide tile is too large for LDS.
  for (int threads : {kConvWideThreads, kConvThreads}) {
    if (!(dx && (dthr || dw)) || !make_tile(g, &t, threads)) continue;
    const int LM = L * int(s.M);
    // channels per workgroup: all of them if that leaves room for a second workgroup on the CU, else a half or a
    // quarter (each window reads the tile's upstream gradient again, which is small beside the walks)
    int c_per = int(s.C);
    ConvLds lay = conv_lds_layout<Real>(t, c_per, V, LM, true, true, true);
    while (lay.total > kConvTiledLdsMax / 2 && c_per >= 16) {  // (at least 8 channels: the lanes' skew spreads over them)
      c_per = (c_per + 1) / 2;
      lay = conv_lds_layout<Real>(t, c_per, V, LM, true, true, true);
    }
    while (lay.total > kConvTiledLdsMax && c_per > 1) {  // ... unless nothing larger fits at all (deep trees)
      c_per = (c_per + 1) / 2;
      lay = conv_lds_layout<Real>(t, c_per, V, LM, true, true, true);
    }
    const long long tiles = t.tiles();
    if (lay.total > kConvTiledLdsMax) continue;
    const int c_blocks = (int(s.C) + c_per - 1) / c_per;
    const int j_per = conv_j_per(tiles * s.B * c_blocks, int(s.Cout));
    const long long grid_y = (long long)((s.Cout + j_per - 1) / j_per) * c_blocks;
    if (grid_y > 65535) continue;
    const dim3 grid((unsigned)tiles, (unsigned)grid_y, (unsigned)s.B);
    auto kernel = fern ? conv_tiled_backward_kernel<Real, true, kConvWideThreads, false>
                       : conv_tiled_backward_kernel<Real, false, kConvWideThreads, false>;
    if (threads == kConvThreads)
      kernel = fern ? conv_tiled_backward_kernel<Real, true, kConvThreads, false>
                    : conv_tiled_backward_kernel<Real, false, kConvThreads, false>;
    if (s.M == 1) {
      kernel = fern ? conv_tiled_backward_kernel<Real, true, kConvWideThreads, true>
                    : conv_tiled_backward_kernel<Real, false, kConvWideThreads, true>;
      if (threads == kConvThreads)
        kernel = fern ? conv_tiled_backward_kernel<Real, true, kConvThreads, true>
                      : conv_tiled_backward_kernel<Real, false, kConvThreads, true>;
    }
    HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));
    hipLaunchKernelGGL(kernel, grid, dim3(threads), lay.total, stream, t, lay, int(s.C), c_per, int(s.Cout),
                       int(s.depth), V, L, int(s.M), j_per, x, thr, ord, w, gout, dx, dthr, dw);
    HT_LAUNCH_CHECK("conv backward (one walk, tiled)");
    return HT_OK;
  }
  if (make_tile(g, &t)) {
    const int LM = L * int(s.M);
    const ConvLds lay_x = conv_lds_layout<Real>(t, int(s.C), V, LM, true, false, true);
    const ConvLds lay_t = conv_lds_layout<Real>(t, int(s.C), V, LM, false, true, true);
    const long long tiles = t.tiles();
    if (lay_x.total <= kConvTiledLdsMax && lay_t.total <= kConvTiledLdsMax) {
      if (dx) {
        const int j_per = conv_j_per(tiles * s.B, int(s.Cout));
        const dim3 grid((unsigned)tiles, (unsigned)((s.Cout + j_per - 1) / j_per), (unsigned)s.B);
        auto kernel = fern ? conv_tiled_dx_kernel<Real, true> : conv_tiled_dx_kernel<Real, false>;
        HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));
        hipLaunchKernelGGL(kernel, grid, dim3(kConvThreads), lay_x.total, stream, t, lay_x, int(s.C), int(s.Cout),
                           int(s.depth), V, L, int(s.M), j_per, x, thr, ord, w, gout, dx);
        HT_LAUNCH_CHECK("conv backward (dX, tiled)");
      }
      if (dthr || dw) {
        const long long items = tiles * s.B;
        long long parts = (4 * kNumCUs + s.Cout - 1) / s.Cout;  // ~4 workgroups per CU
        if (parts > items) parts = items;
        if (parts > 65535) parts = 65535;
        if (parts < 1) parts = 1;
        const dim3 grid((unsigned)s.Cout, (unsigned)parts);
        auto kernel = fern ? conv_tiled_trees_kernel<Real, true> : conv_tiled_trees_kernel<Real, false>;
        HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));
        hipLaunchKernelGGL(kernel, grid, dim3(kConvThreads), lay_t.total, stream, t, lay_t, int(s.C), int(s.Cout),
                           int(s.depth), V, L, int(s.M), items, x, thr, ord, w, gout, dthr, dw);
        HT_LAUNCH_CHECK("conv backward (trees, tiled)");
      }
      return HT_OK;
    }
  }
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
