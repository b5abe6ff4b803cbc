// Dense projection in front of a forest: z = x * lin^T on the matrix cores, batch statistics of z in the same pass,
// normalisation in place, and the matching backward (batch-norm backward + dLin = dz^T * x, dX = dz * lin).
//
// This is the Linear -> BatchNorm1d(affine=False) -> RandomHingeForest composition of the reference's README
// (README.md:117-129, experiments/run_letter_seq.py:45-52) with the two dense stages written for gfx950: the only
// place of this library where MFMA applies. fp32 in, fp32 accumulate (v_mfma_f32_32x32x2_f32).
//
// GEMM tiling: a workgroup of 256 threads (4 wavefronts, 2 x 2) owns a 128 x 128 tile of the result; a wavefront
// owns 64 x 64 of it as 2 x 2 MFMA tiles (64 accumulator registers per lane). The reduction runs in steps of 16:
// both operand tiles are staged in LDS reduction-major (tile[r][i], pitch 132), so the MFMA operand of lane l
// (row l % 32, reduction index l / 32) is one conflict-free ds_read_b32, and the next step's global loads are in
// flight while the current step is multiplied (register double buffering).
#include <type_traits>

#include "common.hpp"
#include "records.hpp"

namespace ht {
namespace {

typedef float Acc16 __attribute__((ext_vector_type(16)));
typedef float Vec4 __attribute__((ext_vector_type(4)));

constexpr int kGemmThreads = 256;
constexpr int kTile = 128;  // result tile edge
constexpr int kRed = 16;    // reduction step
constexpr int kPitch = kTile + 4;

// Operand access patterns. An operand is a [rows x red] matrix that contributes tile[r][i] = op(i0 + i, r0 + r).
//   RED_CONTIG  : element (i, r) at p[i * ld + r]   (reduction index contiguous: x and lin in z = x * lin^T)
//   otherwise   : element (i, r) at p[r * ld + i]   (row index contiguous: dz and x in dLin = dz^T * x)
// Each thread moves 2 x float4 per operand and step.
struct Fetch {
  Vec4 v[2];
};

// `full` (uniform over the workgroup): the whole 128 x 16 tile lies inside the operand and may be read as float4s, so
// no thread needs a bounds check -- the common case, and the one whose instruction count matters.
template <bool RED_CONTIG>
__device__ __forceinline__ void fetch_tile(Fetch &f, const float *__restrict__ p, long long ld, int i0, int n_i,
                                           int r0, int n_r, bool vec_ok, bool full) {
  const int t = threadIdx.x;
  if (full) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const float *src = RED_CONTIG ? p + (long long)(i0 + t / 4 + 64 * h) * ld + r0 + (t % 4) * 4
                                    : p + (long long)(r0 + t / 32 + 8 * h) * ld + i0 + (t % 32) * 4;
      f.v[h] = *reinterpret_cast<const Vec4 *>(src);
    }
    return;
  }
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    Vec4 v = {0.f, 0.f, 0.f, 0.f};
    if (RED_CONTIG) {
      // thread -> (row i = t / 4 + 64 h, reduction quad q = t % 4)
      const int i = i0 + t / 4 + 64 * h, r = r0 + (t % 4) * 4;
      if (i < n_i) {
        const float *src = p + (long long)i * ld + r;
        if (vec_ok && r + 3 < n_r) {
          v = *reinterpret_cast<const Vec4 *>(src);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (r + e < n_r) v[e] = src[e];
        }
      }
    } else {
      // thread -> (reduction index r = t / 32 + 8 h, row quad q = t % 32)
      const int r = r0 + t / 32 + 8 * h, i = i0 + (t % 32) * 4;
      if (r < n_r) {
        const float *src = p + (long long)r * ld + i;
        if (vec_ok && i + 3 < n_i) {
          v = *reinterpret_cast<const Vec4 *>(src);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (i + e < n_i) v[e] = src[e];
        }
      }
    }
    f.v[h] = v;
  }
}

template <bool RED_CONTIG>
__device__ __forceinline__ void stash_tile(float *tile, const Fetch &f) {
  const int t = threadIdx.x;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    if (RED_CONTIG) {
      const int i = t / 4 + 64 * h, r = (t % 4) * 4;
#pragma unroll
      for (int e = 0; e < 4; ++e) tile[(r + e) * kPitch + i] = f.v[h][e];
    } else {
      const int r = t / 32 + 8 * h, i = (t % 32) * 4;
      *reinterpret_cast<Vec4 *>(tile + r * kPitch + i) = f.v[h];
    }
  }
}

// Workgroup -> result tile. Workgroups are dealt to the 8 XCDs (each with its own L2) round robin by index, so
// index % 8 names the L2 a workgroup will use. Every XCD takes a contiguous band of tile rows and walks it in panels
// of 8 tile columns, row by row inside a panel: the ~100 workgroups an XCD runs at a time then cover about 12 x 8
// tiles and share their 12 + 8 operand tiles through that L2, instead of each fetching its own pair.
// Returns false for a launch slot that has no tile (bands are padded to the same number of slots).
__host__ __device__ inline bool gemm_tile_of(int block, int tiles_i, int tiles_j, int rows_per_xcd, int *tile_i,
                                             int *tile_j) {
  const int xcd = block % kNumXCDs, slot = block / kNumXCDs;
  const int row0 = xcd * rows_per_xcd;
  const int rows = rows_per_xcd < tiles_i - row0 ? rows_per_xcd : tiles_i - row0;
  if (rows <= 0 || slot >= rows * tiles_j) return false;
  constexpr int kPanel = 8;
  const int full = tiles_j / kPanel;  // panels of the full width
  int panel = slot / (rows * kPanel), rem = slot - panel * (rows * kPanel), width = kPanel;
  if (panel >= full) {
    panel = full;
    rem = slot - full * (rows * kPanel);
    width = tiles_j - full * kPanel;
  }
  const int r = rem / width;
  *tile_i = row0 + r;
  *tile_j = panel * kPanel + (rem - r * width);
  return true;
}

// C[i, j] = sum_r A(i, r) * B(j, r) (+ bias_i[i] + bias_j[j]), i < n_i, j < n_j, r < n_r; C row-major with leading
// dimension ldc. A launch covers `batches` such problems whose operands lie stride_a / stride_b / stride_c elements
// apart: either one result per batch (blockIdx.z), or -- SUM_BATCHES -- one result summed over all of them (the
// batch index then simply extends the reduction).
// STATS: also accumulate per column j the sum and the sum of squares of C over i into stats[j], stats[n_j + j] (fp64
// atomics; the batch statistics of the projection).
struct GemmArgs {
  const float *A, *B;
  float *C;
  long long lda, ldb, ldc, stride_a, stride_b, stride_c;
  int n_i, n_j, n_r, batches;
  int tiles_i, tiles_j, rows_per_xcd;  // result tiles, and how many tile rows each of the 8 L2 domains takes
  int splits;                          // > 1: blockIdx.y takes a share of the reduction and adds into a zeroed C ...
  long long split_stride;              // ... or, if not 0, stores its share at C + blockIdx.y * split_stride
  bool vec_a, vec_b;
  bool symmetric;  // A and B are the same operand: tiles below the diagonal are not computed but mirrored from above
  double *stats;
  const float *bias_i, *bias_j;
  // A_BN: operand A is not read as it lies in memory but as the batch-norm backward of it, element (i, r) =
  // bn_rstd[i] * (A(i, r) - mean_1[i] - bn_zhat(i, r) * mean_2[i]) with mean_1[i] = bn_sums[i] / bn_count and
  // mean_2[i] = bn_sums[n_i + i] / bn_count (bn_zhat laid out like A)
  const float *bn_zhat, *bn_rstd;
  const double *bn_sums;
  double bn_count;
};

// The batch-norm backward of a fetched operand piece: rstd * (a - mean_1 - zh * mean_2) as two fused multiply-adds,
// a * rstd + (zh * (-rstd * mean_2) + (-rstd * mean_1)) -- a staging step of every reduction step, so its instruction
// count matters; bn_backward_apply_kernel rounds after each of its four operations instead, and the two forms differ
// in the last bits.
// rows: the tile's constants in LDS, [rstd | -rstd * mean_1 | -rstd * mean_2][kTile] (zeros for rows outside the
// operand, which makes their elements zero; in LDS because the kernel has no registers to spare for twelve more values
// per thread); row_ok: the piece's reduction index lies inside the operand (outside, the operand contributes zeros).
__device__ __forceinline__ void bn_backward_piece(Vec4 &a, const Vec4 &zh, const float *rows, bool row_ok) {
  const int i = (int(threadIdx.x) % 32) * 4;
  const Vec4 c0 = *reinterpret_cast<const Vec4 *>(rows + i), c1 = *reinterpret_cast<const Vec4 *>(rows + kTile + i),
             c2 = *reinterpret_cast<const Vec4 *>(rows + 2 * kTile + i);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float v = __builtin_fmaf(a[e], c0[e], __builtin_fmaf(zh[e], c2[e], c1[e]));
    a[e] = row_ok ? v : 0.f;
  }
}

template <bool A_RED_CONTIG, bool B_RED_CONTIG, bool STATS, bool SUM_BATCHES, bool A_BN = false>
__global__ __launch_bounds__(kGemmThreads) __attribute__((amdgpu_waves_per_eu(3, 4))) void gemm_kernel(GemmArgs g) {
  static_assert(!A_BN || (!A_RED_CONTIG && !SUM_BATCHES), "the fused batch-norm backward reads a row-contiguous operand");
  __shared__ float As[2][kRed * kPitch];
  __shared__ float Bs[2][kRed * kPitch];
  const int n_i = g.n_i, n_j = g.n_j, n_r = g.n_r;
  int tile_i, tile_j;
  // A launch slot runs on XCD slot % 8 whatever its share of a split reduction is (the grid's x extent is a multiple
  // of 8), and the tile map gives every XCD a band of tile rows: with few tile rows -- or a symmetric product, whose
  // upper rows hold more tiles -- the shares would pile their work on the same XCDs, so share y takes the band of the
  // XCD y places further on.
  const int slot = int(blockIdx.x) - int(blockIdx.x) % kNumXCDs + (int(blockIdx.x) + int(blockIdx.y)) % kNumXCDs;
  if (!gemm_tile_of(slot, g.tiles_i, g.tiles_j, g.rows_per_xcd, &tile_i, &tile_j)) return;
  if (g.symmetric && tile_j < tile_i) return;
  const int i0 = tile_i * kTile, j0 = tile_j * kTile;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wi = (wave >> 1) * 64, wj = (wave & 1) * 64;  // this wavefront's 64 x 64 corner
  const int lr = lane & 31, lk = lane >> 5;
  const float *A = g.A, *B = g.B;
  float *C = g.C + (long long)blockIdx.y * g.split_stride;
  if (!SUM_BATCHES) {
    A += (long long)blockIdx.z * g.stride_a;
    B += (long long)blockIdx.z * g.stride_b;
    C += (long long)blockIdx.z * g.stride_c;
  }

  Acc16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;

  const int per_batch = (n_r + kRed - 1) / kRed;
  // this workgroup's share of the reduction steps (all of them unless the launch splits the reduction)
  const int all_steps = SUM_BATCHES ? per_batch * g.batches : per_batch;
  const int chunk = (all_steps + g.splits - 1) / g.splits;
  const int step0 = blockIdx.y * chunk;
  const int steps = max(0, min(chunk, all_steps - step0));
  if (g.splits > 1 && steps == 0) return;
  const bool rows_a_full = g.vec_a && i0 + kTile <= n_i, rows_b_full = g.vec_b && j0 + kTile <= n_j;
  __shared__ __align__(16) float bn[A_BN ? 3 * kTile : 4];
  if constexpr (A_BN) {
    if (threadIdx.x < kTile) {
      const int i = i0 + int(threadIdx.x);
      const bool in = i < n_i;
      const float rstd = in ? g.bn_rstd[i] : 0.f;
      bn[threadIdx.x] = rstd;
      bn[kTile + threadIdx.x] = in ? -rstd * float(g.bn_sums[i] / g.bn_count) : 0.f;
      bn[2 * kTile + threadIdx.x] = in ? -rstd * float(g.bn_sums[n_i + i] / g.bn_count) : 0.f;
    }
    __syncthreads();
  }
  // Pipeline: while step s is multiplied out of LDS buffer s & 1, the operands of step s + 1 (fetched during step
  // s - 1) are written to the other buffer in the middle of the multiply, and the global loads of step s + 2 are in
  // flight. A wavefront therefore issues its LDS writes and address arithmetic in the shadow of its own MFMAs, and one
  // barrier per step remains.
  // 32-wide blocks of this wavefront's corner that hold any result at all (wave uniform). In a tile on the ragged edge
  // of the result the others are skipped: a dLin of 784 columns ends in a tile column with 16 of them, where one
  // wavefront in two has nothing to multiply and the other one block column instead of two.
  const int na = __builtin_amdgcn_readfirstlane(max(0, min(2, (n_i - i0 - wi + 31) / 32)));
  const int nb = __builtin_amdgcn_readfirstlane(max(0, min(2, (n_j - j0 - wj + 31) / 32)));
  auto multiply = [&](const float *as, const float *bs, int kk_begin, int kk_end, auto edge_tag) {
    constexpr bool EDGE = decltype(edge_tag)::value;
#pragma unroll
    for (int kk = kk_begin; kk < kk_end; kk += 2) {
      const float a0 = as[(kk + lk) * kPitch + wi + lr], a1 = as[(kk + lk) * kPitch + wi + 32 + lr];
      const float b0 = bs[(kk + lk) * kPitch + wj + lr], b1 = bs[(kk + lk) * kPitch + wj + 32 + lr];
      if (!EDGE || (na > 0 && nb > 0)) acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
      if (!EDGE || (na > 0 && nb > 1)) acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
      if (!EDGE || (na > 1 && nb > 0)) acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
      if (!EDGE || (na > 1 && nb > 1)) acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
    }
  };
  // The loop exists twice: for workgroups whose operand tiles all lie inside the matrices (FULL: exactly four
  // unconditional float4 loads per fetch, so the wait in front of the LDS writes can leave the newest four in flight)
  // and for the edge tiles (bounds checks, a data-dependent number of loads, hence full waits).
  auto run = [&](auto full_tag) {
    constexpr bool FULL = decltype(full_tag)::value;
    // (A_BN: an operand piece of A travels with the matching piece of zhat, in the second half of the same structure)
    struct FetchA {
      Fetch a, zh;
    };
    auto fetch = [&](FetchA &fa, Fetch &fb, int s) {
      const int gs = s + step0;
      const int z = SUM_BATCHES ? gs / per_batch : 0;
      const int r0 = (gs - z * per_batch) * kRed;
      fetch_tile<A_RED_CONTIG>(fa.a, A + (long long)z * g.stride_a, g.lda, i0, n_i, r0, n_r, g.vec_a, FULL);
      if constexpr (A_BN) fetch_tile<false>(fa.zh, g.bn_zhat, g.lda, i0, n_i, r0, n_r, g.vec_a, FULL);
      fetch_tile<B_RED_CONTIG>(fb, B + (long long)z * g.stride_b, g.ldb, j0, n_j, r0, n_r, g.vec_b, FULL);
    };
    // operands of step s from registers into an LDS buffer
    auto stash = [&](int buffer, FetchA &fa, const Fetch &fb, int s) {
      if constexpr (A_BN) {
        const int r0 = (s + step0) * kRed;
#pragma unroll
        for (int h = 0; h < 2; ++h)
          bn_backward_piece(fa.a.v[h], fa.zh.v[h], bn, FULL || r0 + int(threadIdx.x) / 32 + 8 * h < n_r);
      }
      stash_tile<A_RED_CONTIG>(As[buffer], fa.a);
      stash_tile<B_RED_CONTIG>(Bs[buffer], fb);
    };
    if constexpr (A_BN) {
      // One step of lookahead only: the operands of step s + 1 are requested when step s begins and written to LDS
      // when its products are done. With zhat travelling beside A, two steps in flight need more registers than three
      // wavefronts per SIMD leave, and the third wavefront hides more latency than the second step ahead did.
      FetchA fa;
      Fetch fb;
      if (steps > 0) {
        fetch(fa, fb, 0);
        stash(0, fa, fb, 0);
      }
      __syncthreads();
      for (int s = 0; s < steps; ++s) {
        const int cur = s & 1;
        const bool more = s + 1 < steps;
        if (more) fetch(fa, fb, s + 1);
        multiply(As[cur], Bs[cur], 0, kRed, std::integral_constant<bool, !FULL>{});
        if (more) stash(cur ^ 1, fa, fb, s + 1);
        __syncthreads();
      }
      return;
    }
    FetchA fa0, fa1;
    Fetch fb0, fb1;
    if (steps > 0) {
      fetch(fa0, fb0, 0);
      stash(0, fa0, fb0, 0);
      if (steps > 1) fetch(fa0, fb0, 1);
    }
    __syncthreads();
    // one step: `held` carries the operands of step s + 1, `next` receives those of step s + 2. PREFETCH is a
    // compile-time property of the call site: the steady-state loop always fetches (so the wait in front of the LDS
    // writes may leave exactly those newest loads in flight), the last two steps never do.
    auto step = [&](int s, FetchA &held_a, Fetch &held_b, FetchA &next_a, Fetch &next_b, auto prefetch_tag) {
      constexpr bool PREFETCH = decltype(prefetch_tag)::value;
      const int cur = s & 1;
      if (PREFETCH) fetch(next_a, next_b, s + 2);
      multiply(As[cur], Bs[cur], 0, kRed / 2, std::integral_constant<bool, !FULL>{});
      if (PREFETCH || s + 1 < steps) stash(cur ^ 1, held_a, held_b, s + 1);
      multiply(As[cur], Bs[cur], kRed / 2, kRed, std::integral_constant<bool, !FULL>{});
      __syncthreads();
    };
    int s = 0;
    for (; s + 3 < steps; s += 2) {  // both steps have a step s + 2 to fetch
      step(s, fa0, fb0, fa1, fb1, std::true_type{});
      step(s + 1, fa1, fb1, fa0, fb0, std::true_type{});
    }
    if (s + 2 < steps) {             // one more step that fetches; the operand registers swap roles once more
      step(s, fa0, fb0, fa1, fb1, std::true_type{});
      step(s + 1, fa1, fb1, fa0, fb0, std::false_type{});
      step(s + 2, fa0, fb0, fa1, fb1, std::false_type{});
    } else {
      if (s < steps) step(s, fa0, fb0, fa1, fb1, std::false_type{});
      if (s + 1 < steps) step(s + 1, fa1, fb1, fa0, fb0, std::false_type{});
    }
  };
  if (rows_a_full && rows_b_full && n_r % kRed == 0)
    run(std::true_type{});
  else
    run(std::false_type{});

  // accumulator element e of lane l is C(row 8 * (e / 4) + 4 * (l / 32) + e % 4, column l % 32) of its 32 x 32 tile
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    const int j = j0 + wj + 32 * b + lr;
    const bool first = blockIdx.y == 0;  // the biases belong to one share of a split reduction only
    const float bj = (g.bias_j && first && j < n_j) ? g.bias_j[j] : 0.f;
    double s1 = 0.0, s2 = 0.0;
#pragma unroll
    for (int a = 0; a < 2; ++a) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int i = i0 + wi + 32 * a + 8 * (e / 4) + 4 * lk + (e % 4);
        if (i < n_i && j < n_j) {
          float v = acc[a][b][e];
          if (g.bias_i && first) v += g.bias_i[i];
          v += bj;
          if (g.splits > 1 && g.split_stride == 0) {
            atomicAdd(C + (long long)i * g.ldc + j, v);
          } else {
            C[(long long)i * g.ldc + j] = v;
            if (g.symmetric && tile_i != tile_j) C[(long long)j * g.ldc + i] = v;
          }
          if (STATS) {
            s1 += double(v);
            s2 += double(v) * double(v);
          }
        }
      }
    }
    if (STATS) {
      s1 += __shfl_xor(s1, 32, 64);
      s2 += __shfl_xor(s2, 32, 64);
      if (lk == 0 && j < n_j) {
        atomicAdd(g.stats + j, s1);
        atomicAdd(g.stats + n_j + j, s2);
      }
    }
  }
}

// mean, rstd (and the biased variance) of every column from the accumulated sums.
__global__ void bn_finalize_kernel(const double *__restrict__ stats, int N, long long B, double eps, float *mean,
                                   float *rstd, float *var) {
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= N) return;
  const double m = stats[j] / double(B);
  double v = stats[N + j] / double(B) - m * m;
  if (v < 0.0) v = 0.0;
  mean[j] = float(m);
  rstd[j] = float(1.0 / sqrt(v + eps));
  if (var) var[j] = float(v);
}

// z <- (z - mean) * rstd, in place, row-major [B x N]. One thread per 4 consecutive columns of 8 rows.
__global__ __launch_bounds__(256) void bn_apply_kernel(float *z, long long B, int N, const float *__restrict__ mean,
                                                       const float *__restrict__ rstd) {
  const int j = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (j >= N) return;
  float m[4], r[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    m[e] = j + e < N ? mean[j + e] : 0.f;
    r[e] = j + e < N ? rstd[j + e] : 0.f;
  }
  const bool vec = (N % 4 == 0) && (reinterpret_cast<uintptr_t>(z) % 16 == 0);
  for (long long i = blockIdx.y; i < B; i += gridDim.y) {
    float *p = z + i * N + j;
    if (vec) {
      Vec4 v = *reinterpret_cast<Vec4 *>(p);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (v[e] - m[e]) * r[e];
      *reinterpret_cast<Vec4 *>(p) = v;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (j + e < N) p[e] = (p[e] - m[e]) * r[e];
    }
  }
}

// Column sums of g and of g * zhat over the rows (fp64 atomics into sums[j], sums[N + j]).
__global__ __launch_bounds__(256) void bn_backward_sums_kernel(const float *__restrict__ g,
                                                               const float *__restrict__ zhat, long long B, int N,
                                                               double *sums) {
  const int j = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (j >= N) return;
  double s1[4] = {0, 0, 0, 0}, s2[4] = {0, 0, 0, 0};
  const bool vec = (N % 4 == 0) && (reinterpret_cast<uintptr_t>(g) % 16 == 0) &&
                   (reinterpret_cast<uintptr_t>(zhat) % 16 == 0);
  for (long long i = blockIdx.y; i < B; i += gridDim.y) {
    float gv[4], zv[4];
    if (vec) {
      const Vec4 a = *reinterpret_cast<const Vec4 *>(g + i * N + j), b = *reinterpret_cast<const Vec4 *>(zhat + i * N + j);
#pragma unroll
      for (int e = 0; e < 4; ++e) gv[e] = a[e], zv[e] = b[e];
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        gv[e] = j + e < N ? g[i * N + j + e] : 0.f;
        zv[e] = j + e < N ? zhat[i * N + j + e] : 0.f;
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      s1[e] += double(gv[e]);
      s2[e] += double(gv[e]) * double(zv[e]);
    }
  }
#pragma unroll
  for (int e = 0; e < 4; ++e)
    if (j + e < N) {
      atomicAdd(sums + j + e, s1[e]);
      atomicAdd(sums + N + j + e, s2[e]);
    }
}

// g <- rstd * (g - mean(g) - zhat * mean(g * zhat)), in place (batch-norm backward without affine parameters).
__global__ __launch_bounds__(256) void bn_backward_apply_kernel(float *g, const float *__restrict__ zhat, long long B,
                                                                int N, const float *__restrict__ rstd,
                                                                const double *__restrict__ sums) {
  const int j = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (j >= N) return;
  float r[4], m1[4], m2[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const bool in = j + e < N;
    r[e] = in ? rstd[j + e] : 0.f;
    m1[e] = in ? float(sums[j + e] / double(B)) : 0.f;
    m2[e] = in ? float(sums[N + j + e] / double(B)) : 0.f;
  }
  const bool vec = (N % 4 == 0) && (reinterpret_cast<uintptr_t>(g) % 16 == 0) &&
                   (reinterpret_cast<uintptr_t>(zhat) % 16 == 0);
  for (long long i = blockIdx.y; i < B; i += gridDim.y) {
    float *p = g + i * N + j;
    const float *q = zhat + i * N + j;
    if (vec) {
      Vec4 a = *reinterpret_cast<Vec4 *>(p);
      const Vec4 b = *reinterpret_cast<const Vec4 *>(q);
#pragma unroll
      for (int e = 0; e < 4; ++e) a[e] = r[e] * (a[e] - m1[e] - b[e] * m2[e]);
      *reinterpret_cast<Vec4 *>(p) = a;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (j + e < N) p[e] = r[e] * (p[e] - m1[e] - q[e] * m2[e]);
    }
  }
}

constexpr long long kMaxGridZ = 65535;  // limit of gridDim.z

// dst[i] = shares[0][i] + shares[1][i] + ... in that order (n elements per share).
__global__ __launch_bounds__(256) void sum_shares_kernel(const float *__restrict__ shares, int count, long long n,
                                                         float *dst) {
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
    float v = shares[i];
    for (int s = 1; s < count; ++s) v += shares[(long long)s * n + i];
    dst[i] = v;
  }
}

bool aligned16(const void *p, long long ld, long long stride) {
  return reinterpret_cast<uintptr_t>(p) % 16 == 0 && ld % 4 == 0 && stride % 4 == 0;
}

// The batch-norm backward that a product applies to its operand A while loading it (see GemmArgs).
struct BnOperand {
  const float *zhat, *rstd;
  const double *sums;
  double count;
};

template <bool A_RED_CONTIG, bool B_RED_CONTIG, bool STATS, bool SUM_BATCHES, bool A_BN = false>
int launch_gemm_batched(const float *A, long long lda, long long stride_a, const float *B, long long ldb,
                        long long stride_b, float *C, long long ldc, long long stride_c, long long n_i, long long n_j,
                        long long n_r, long long batches, double *stats, const float *bias_i, const float *bias_j,
                        hipStream_t stream, bool allow_split = false, float *partials = nullptr, int ordered_splits = 0,
                        const BnOperand *bn = nullptr, bool symmetric = false) {
  if (n_i <= 0 || n_j <= 0 || batches <= 0) return HT_OK;
  if (!SUM_BATCHES && batches > kMaxGridZ) {
    // one result per batch rides on blockIdx.z: longer batch lists go out in several launches
    for (long long b0 = 0; b0 < batches; b0 += kMaxGridZ) {
      const long long nb = batches - b0 < kMaxGridZ ? batches - b0 : kMaxGridZ;
      int rc = launch_gemm_batched<A_RED_CONTIG, B_RED_CONTIG, STATS, SUM_BATCHES, false>(
          A + b0 * stride_a, lda, stride_a, B + b0 * stride_b, ldb, stride_b, C + b0 * stride_c, ldc, stride_c, n_i, n_j,
          n_r, nb, stats, bias_i, bias_j, stream, allow_split);
      if (rc != HT_OK) return rc;
    }
    return HT_OK;
  }
  const long long gi = (n_i + kTile - 1) / kTile, gj = (n_j + kTile - 1) / kTile;
  const long long per_batch = (n_r + kRed - 1) / kRed;
  if (gi > 0x7fffffffLL || gj > 0x7fffffffLL || n_r > 0x7fffffffLL || n_i > 0x7fffffffLL || n_j > 0x7fffffffLL ||
      batches > 0x7fffffffLL || per_batch * batches > 0x7fffffffLL)
    return fail(HT_ERR_RUNTIME, "Error: matrix product too large for this build.");
  GemmArgs g;
  g.A = A, g.B = B, g.C = C;
  g.lda = lda, g.ldb = ldb, g.ldc = ldc;
  g.stride_a = stride_a, g.stride_b = stride_b, g.stride_c = stride_c;
  g.n_i = int(n_i), g.n_j = int(n_j), g.n_r = int(n_r), g.batches = int(batches);
  g.tiles_i = int(gi), g.tiles_j = int(gj), g.rows_per_xcd = int((gi + kNumXCDs - 1) / kNumXCDs);
  const long long slots = (long long)g.rows_per_xcd * gj * kNumXCDs;
  if (slots > 0x7fffffffLL) return fail(HT_ERR_RUNTIME, "Error: matrix product too large for this build.");
  g.vec_a = aligned16(A, lda, stride_a), g.vec_b = aligned16(B, ldb, stride_b);
  g.stats = stats, g.bias_i = bias_i, g.bias_j = bias_j;
  // (mirrored stores are plain stores: not with atomic shares, statistics or biases)
  g.symmetric = symmetric && A == B && lda == ldb && n_i == n_j && ldc == n_j && !STATS && !bias_i && !bias_j && batches == 1;
  g.bn_zhat = g.bn_rstd = nullptr, g.bn_sums = nullptr, g.bn_count = 1.0;
  if (A_BN) {
    if (!bn || batches != 1) return fail(HT_ERR_RUNTIME, "Error: fused batch-norm operand needs its statistics.");
    g.bn_zhat = bn->zhat, g.bn_rstd = bn->rstd, g.bn_sums = bn->sums, g.bn_count = bn->count;
    g.vec_a = g.vec_a && aligned16(bn->zhat, lda, 0);
  }
  // A product with few result tiles and a long reduction (dLin of a narrow linear head: 10 x 1000 from 65536 rows)
  // would leave most of the device idle: the reduction is then split over blockIdx.y and the shares are added into
  // the zeroed result with float atomics (a few thousand elements times the number of shares).
  g.splits = 1;
  g.split_stride = 0;
  const long long all_steps = SUM_BATCHES ? per_batch * batches : per_batch;
  if (ordered_splits > 1 && partials != nullptr && !STATS && ldc == n_j && batches == 1 && !bias_i && !bias_j) {
    // reproducible form of the split: every share stores its partial result, and the shares are added in a fixed order
    g.splits = ordered_splits;
    g.split_stride = n_i * n_j;
    g.C = partials;
    hipLaunchKernelGGL((gemm_kernel<A_RED_CONTIG, B_RED_CONTIG, STATS, SUM_BATCHES, A_BN>),
                       dim3((unsigned)slots, (unsigned)g.splits, 1u), dim3(kGemmThreads), 0, stream, g);
    HT_LAUNCH_CHECK("matrix product (matrix cores, split reduction)");
    const long long chunk = (all_steps + g.splits - 1) / g.splits;
    const int filled = int((all_steps + chunk - 1) / chunk);  // shares that had steps to do (the others wrote nothing)
    const long long n = n_i * n_j;
    hipLaunchKernelGGL(sum_shares_kernel, dim3((unsigned)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192)), dim3(256), 0,
                       stream, partials, filled, n, C);
    HT_LAUNCH_CHECK("matrix product (sum of the shares)");
    return HT_OK;
  }
  if (allow_split) g.symmetric = false;
  if (allow_split && !STATS && ldc == n_j && (SUM_BATCHES || batches == 1) && gi * gj < kNumCUs && all_steps >= 64) {
    long long want = (2 * kNumCUs + gi * gj - 1) / (gi * gj);
    if (want > all_steps / 16) want = all_steps / 16;
    if (want > 65535) want = 65535;
    if (want > 1) {
      g.splits = int(want);
      int rc = zero_fill(C, size_t(n_i) * size_t(n_j) * sizeof(float), stream);
      if (rc != HT_OK) return rc;
    }
  }
  hipLaunchKernelGGL((gemm_kernel<A_RED_CONTIG, B_RED_CONTIG, STATS, SUM_BATCHES, A_BN>),
                     dim3((unsigned)slots, (unsigned)g.splits, (unsigned)(SUM_BATCHES ? 1 : batches)), dim3(kGemmThreads),
                     0, stream, g);
  HT_LAUNCH_CHECK("matrix product (matrix cores)");
  return HT_OK;
}

template <bool A_RED_CONTIG, bool B_RED_CONTIG, bool STATS>
int launch_gemm(const float *A, long long lda, const float *B, long long ldb, float *C, long long ldc, long long n_i,
                long long n_j, long long n_r, double *stats, hipStream_t stream) {
  return launch_gemm_batched<A_RED_CONTIG, B_RED_CONTIG, STATS, false>(A, lda, 0, B, ldb, 0, C, ldc, 0, n_i, n_j, n_r, 1,
                                                                        stats, nullptr, nullptr, stream);
}

long long rows_grid(long long B) { return B < 64 ? (B < 1 ? 1 : B) : 64; }

}  // namespace

int gemm_tile_map(int tiles_i, int tiles_j, int *tile_i, int *tile_j) {
  const int rows_per_xcd = (tiles_i + kNumXCDs - 1) / kNumXCDs;
  const long long slots = (long long)rows_per_xcd * tiles_j * kNumXCDs;
  for (long long b = 0; b < slots; ++b)
    if (!gemm_tile_of(int(b), tiles_i, tiles_j, rows_per_xcd, &tile_i[b], &tile_j[b])) tile_i[b] = tile_j[b] = -1;
  return int(slots);
}

size_t projection_workspace(long long N) { return align_up(size_t(2) * size_t(N) * sizeof(double), 256); }

// Shares of the reduction of a product with rows x cols results over `red` terms (1: no split): long reductions whose
// result tiles do not fill the device evenly by themselves.
int reduction_shares(long long rows, long long cols, long long red) {
  const long long tiles = ((rows + kTile - 1) / kTile) * ((cols + kTile - 1) / kTile), steps = (red + kRed - 1) / kRed;
  if (tiles <= 0 || steps < 64) return 1;
  long long want;
  if (tiles < kNumCUs / 2) {
    // a handful of tiles: enough shares to put four workgroups on every CU (a workgroup alone on a CU waits out every
    // operand latency by itself: xc^T xc of the README model, 49 tiles over 16 384 rows, 0.32 ms with 11 shares)
    want = (4 * kNumCUs + tiles - 1) / tiles;
    if (want > steps / 16) want = steps / 16;
  } else {
    // A few tiles per CU: tiles are equal pieces of work, so 700 of them leave some CUs with three and some with two
    // while the product takes as long as three. About twenty pieces per CU level that out (the README model's dLin,
    // 100 x 7 tiles over 16 384 rows: backward pass 4.22 ms with one share, 3.90 with six, 3.79 with eight, 3.86 with
    // sixteen, the sum of the shares included), each still a reduction of 64 steps or more and all of them together
    // within a GiB of partial results.
    want = (20 * kNumCUs + tiles - 1) / tiles;
    if (want > steps / 64) want = steps / 64;
    const long long bytes = rows * cols * (long long)sizeof(float);
    if (bytes > 0 && want > (1LL << 30) / bytes) want = (1LL << 30) / bytes;
  }
  return want > 1 ? int(want) : 1;
}
// dLin [N x K] reduces over the batch, dX [B x K] over the N columns; the two products run one after the other and
// share the area for their partial results.
size_t shares_bytes(long long B, long long K, long long N) {
  const int s_lin = reduction_shares(N, K, B), s_x = reduction_shares(B, K, N);
  const size_t lin = s_lin > 1 ? size_t(s_lin) * size_t(N) * size_t(K) * sizeof(float) : 0;
  const size_t dx = s_x > 1 ? size_t(s_x) * size_t(B) * size_t(K) * sizeof(float) : 0;
  return lin > dx ? lin : dx;
}

size_t projection_backward_workspace(long long B, long long K, long long N) {
  return projection_workspace(N) + shares_bytes(B, K, N);
}

// zhat [B x N] = normalised (x [B x K] * lin [N x K]^T); mean, rstd, var [N] out; ws: projection_workspace(N).
int projection_forward(long long B, long long K, long long N, const float *x, const float *lin, double eps,
                       float *zhat, float *mean, float *rstd, float *var, void *ws, hipStream_t stream) {
  int rc;
  double *stats = static_cast<double *>(ws);
  if ((rc = zero_fill(stats, size_t(2) * N * sizeof(double), stream)) != HT_OK) return rc;
  if (B == 0 || N == 0) return HT_OK;
  if ((rc = launch_gemm<true, true, true>(x, K, lin, K, zhat, N, B, N, K, stats, stream)) != HT_OK) return rc;
  hipLaunchKernelGGL(bn_finalize_kernel, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, stream, stats, int(N), B, eps,
                     mean, rstd, var);
  HT_LAUNCH_CHECK("batch statistics");
  hipLaunchKernelGGL(bn_apply_kernel, dim3((unsigned)((N + 1023) / 1024), (unsigned)rows_grid(B)), dim3(256), 0, stream,
                     zhat, B, int(N), mean, rstd);
  HT_LAUNCH_CHECK("normalisation");
  return HT_OK;
}

// g [B x N] holds dL/dzhat on entry; where dx is wanted it holds dL/dz on return, otherwise it is left as it came.
// dlin [N x K] and / or dx [B x K] out (either may be null).
int projection_backward(long long B, long long K, long long N, const float *x, const float *lin, const float *zhat,
                        const float *rstd, float *g, float *dlin, float *dx, void *ws, hipStream_t stream) {
  int rc;
  double *sums = static_cast<double *>(ws);
  if ((rc = zero_fill(sums, size_t(2) * N * sizeof(double), stream)) != HT_OK) return rc;
  if (B == 0 || N == 0) {
    if (dlin && (rc = zero_fill(dlin, size_t(N) * K * sizeof(float), stream)) != HT_OK) return rc;
    if (dx && (rc = zero_fill(dx, size_t(B) * K * sizeof(float), stream)) != HT_OK) return rc;
    return HT_OK;
  }
  const dim3 grid((unsigned)((N + 1023) / 1024), (unsigned)rows_grid(B));
  hipLaunchKernelGGL(bn_backward_sums_kernel, grid, dim3(256), 0, stream, g, zhat, B, int(N), sums);
  HT_LAUNCH_CHECK("batch-norm backward (sums)");
  float *partials = reinterpret_cast<float *>(static_cast<unsigned char *>(ws) + projection_workspace(N));
  if (dlin && !dx) {
    // dLin alone, the training case of a first layer: dL/dz is not written out and read back, the product's loader
    // turns dL/dzhat into it on the way into LDS (same arithmetic, same dLin bit for bit); g stays as it came
    const BnOperand bn = {zhat, rstd, sums, double(B)};
    return launch_gemm_batched<false, false, false, false, true>(g, N, 0, x, K, 0, dlin, K, 0, N, K, B, 1, nullptr, nullptr,
                                                                  nullptr, stream, false, partials,
                                                                  reduction_shares(N, K, B), &bn);
  }
  hipLaunchKernelGGL(bn_backward_apply_kernel, grid, dim3(256), 0, stream, g, zhat, B, int(N), rstd, sums);
  HT_LAUNCH_CHECK("batch-norm backward");
  // dlin[n, k] = sum_b g[b, n] * x[b, k]: both operands row contiguous, reduction over the batch. A small layer under a
  // large batch has a handful of result tiles and a long reduction: it is then split over workgroups whose shares are
  // summed in a fixed order (reproducible, unlike a split that meets in atomics).
  if (dlin && (rc = launch_gemm_batched<false, false, false, false>(g, N, 0, x, K, 0, dlin, K, 0, N, K, B, 1, nullptr,
                                                                     nullptr, nullptr, stream, false, partials,
                                                                     reduction_shares(N, K, B))) != HT_OK)
    return rc;
  // dx[b, k] = sum_n g[b, n] * lin[n, k]: g has the reduction index n contiguous, lin the row index k (split the same
  // way where a small batch meets a wide layer)
  if (dx && (rc = launch_gemm_batched<true, false, false, false>(g, N, 0, lin, K, 0, dx, K, 0, B, K, N, 1, nullptr,
                                                                  nullptr, nullptr, stream, false, partials,
                                                                  reduction_shares(B, K, N))) != HT_OK)
    return rc;
  return HT_OK;
}

namespace {

// ---- dLin of Linear -> BatchNorm(affine = False) -> forest, from the forest's walk records ------------------------
//
// The upstream gradient of the normalisation, g = dL/dzhat [B x N], is the forest's dX: one non-zero per (sample, tree)
// pair -- c at the feature the selected vertex looks at -- so B * T entries out of B * N (1.6 M of 208 M for the README
// model). Instead of writing that matrix densely, summing its columns, normalising it and multiplying it by x as a dense
// 2 * B * N * K product, the gradient is taken apart:
//   dz = rstd * (g - m1 - zhat * m2),  m1 = mean_b g,  m2 = mean_b (g * zhat)            (batch-norm backward)
//   dLin[n, k] = sum_b dz[b, n] * x[b, k]
//              = rstd[n] * (sum_b g[b, n] * xc[b, k]  -  m2[n] * sum_b zhat[b, n] * xc[b, k])
// with xc = x - mean_b x: the m1 term vanishes against the centring (sum_b xc = 0), and centring costs nothing on the
// zhat term because sum_b zhat = 0. The second sum is rstd[n] * (lin * Gc)[n, k] with Gc = xc^T xc [K x K], since
// zhat = (x lin^T - mean) * rstd: two small dense products (2 B K^2 + 2 N K^2 operations instead of 2 B N K).
// The first sum is sparse: per (tree, vertex) the rows of xc of the samples that selected it, weighted by c. No term is
// a difference of large numbers. m2 is sparse as well: c * zhat at the selected feature.
//
// Steps: column means of x and xc; per tree the samples bucketed by selected vertex (counting sort in LDS); one
// wavefront per (tree, vertex) segment sums c * xc rows in registers (lanes along K) and c * zhat; the two products on
// the matrix cores; an elementwise combination. The order of a segment's samples depends on scheduling (bucket cursors
// are LDS atomics), so like every atomic-mode gradient the last bits can differ between runs.

constexpr int kBucketThreads = 1024;
constexpr int kMaxBucketVertices = 16384;  // LDS counters of the bucketing kernel

// sums[k] += sum_b x[b, k] (fp64 atomics). A workgroup takes 64 column quads x a share of the rows, its four wavefronts
// alternate rows and meet in LDS: one atomic per column and workgroup.
__global__ __launch_bounds__(256) void col_sums_kernel(const float *__restrict__ x, long long B, int K, double *sums) {
  __shared__ double part[3][kWave][4];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int k = (blockIdx.x * kWave + lane) * 4;
  double s[4] = {0, 0, 0, 0};
  if (k < K)
    for (long long b = (long long)blockIdx.y * 4 + wave; b < B; b += (long long)gridDim.y * 4) {
      const Vec4 v = *reinterpret_cast<const Vec4 *>(x + b * K + k);
#pragma unroll
      for (int e = 0; e < 4; ++e) s[e] += double(v[e]);
    }
  if (wave > 0)
#pragma unroll
    for (int e = 0; e < 4; ++e) part[wave - 1][lane][e] = s[e];
  __syncthreads();
  if (wave == 0 && k < K)
#pragma unroll
    for (int e = 0; e < 4; ++e) atomicAdd(sums + k + e, s[e] + part[0][lane][e] + part[1][lane][e] + part[2][lane][e]);
}

// xc[b, k] = x[b, k] - float(sums[k] / B)
__global__ __launch_bounds__(256) void center_kernel(const float *__restrict__ x, long long B, int K,
                                                     const double *__restrict__ sums, float *__restrict__ xc) {
  const int k = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (k >= K) return;
  float m[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) m[e] = float(sums[k + e] / double(B));
  for (long long b = blockIdx.y; b < B; b += gridDim.y) {
    Vec4 v = *reinterpret_cast<const Vec4 *>(x + b * K + k);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] -= m[e];
    *reinterpret_cast<Vec4 *>(xc + b * K + k) = v;
  }
}

// One workgroup per tree: the tree's S samples ordered by the vertex they selected, as sample indices in perm[t][.].
template <bool COMPACT>
__global__ __launch_bounds__(kBucketThreads) void bucket_kernel(ForestDims d, Records<float, COMPACT> rec,
                                                                uint32_t *__restrict__ perm) {
  extern __shared__ __align__(16) unsigned char smem[];
  uint32_t *count = reinterpret_cast<uint32_t *>(smem);  // [V], then the segments' cursors
  __shared__ uint32_t wave_total[kBucketThreads / kWave];
  const int t = blockIdx.x;
  const long long first = (long long)t * d.S;
  for (int v = threadIdx.x; v < d.V; v += kBucketThreads) count[v] = 0u;
  __syncthreads();
  for (long long s = threadIdx.x; s < d.S; s += kBucketThreads) atomicAdd(&count[min(rec.vertex(first + s), uint32_t(d.V - 1))], 1u);
  __syncthreads();
  // exclusive scan over the V counters: a thread owns a run of `per` consecutive ones
  const int per = (d.V + kBucketThreads - 1) / kBucketThreads;
  const int v0 = min(int(threadIdx.x) * per, d.V), v1 = min(v0 + per, d.V);
  uint32_t mine = 0u;
  for (int v = v0; v < v1; ++v) mine += count[v];
  uint32_t scan = mine;  // inclusive over the wavefront
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  for (int off = 1; off < kWave; off <<= 1) {
    const uint32_t o = __shfl_up(scan, off, kWave);
    if (lane >= off) scan += o;
  }
  if (lane == kWave - 1) wave_total[wave] = scan;
  __syncthreads();
  uint32_t before = scan - mine;
  for (int wv = 0; wv < wave; ++wv) before += wave_total[wv];
  __syncthreads();
  for (int v = v0; v < v1; ++v) {
    const uint32_t n = count[v];
    count[v] = before;
    before += n;
  }
  __syncthreads();
  for (long long s = threadIdx.x; s < d.S; s += kBucketThreads) {
    const uint32_t at = atomicAdd(&count[min(rec.vertex(first + s), uint32_t(d.V - 1))], 1u);
    perm[first + at] = uint32_t(s);
  }
}

constexpr int kSegmentQuads = 4;  // float4 accumulators per lane: 1024 columns per pass over a block
constexpr int kSegmentRows = 4;   // rows of xc requested together

// One wavefront per (tree, block of 64 entries of the tree's vertex-ordered sample list): acc[n, :] += sum_i c_i *
// xc[s_i, :] and m2sum[n] += sum_i c_i * zhat[s_i, n], n the feature the entries' vertex looks at. A lane first takes one
// entry (sample index, c, vertex, feature, c * zhat); the block falls into runs of equal vertices (the list is ordered
// by vertex), and run by run every entry's row of xc is read by the whole wavefront, lanes along the row, four rows in
// flight, and summed in registers; a run ends in atomic adds on its feature's row of acc (a run is a piece of a
// segment: vertices that many samples select spread over many wavefronts instead of one long serial loop).
template <bool COMPACT>
__global__ __launch_bounds__(256) void segment_sums_kernel(ForestDims d, Records<float, COMPACT> rec,
                                                           const float *__restrict__ c,
                                                           const uint32_t *__restrict__ perm,
                                                           const float *__restrict__ xc, int K,
                                                           const float *__restrict__ zhat,
                                                           const float *__restrict__ z_mean,
                                                           const float *__restrict__ z_rstd, float *acc_out,
                                                           double *m2sum) {
  const int lane = threadIdx.x & (kWave - 1);
  const long long blocks_per_tree = (d.S + kWave - 1) / kWave;
  const long long id = (long long)blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
  if (id >= (long long)d.T * blocks_per_tree) return;
  const int t = int(id / blocks_per_tree);
  const long long i0 = (id - (long long)t * blocks_per_tree) * kWave;
  const int count = int(min<long long>(kWave, d.S - i0));
  const long long first = (long long)t * d.S;
  uint32_t s_mine = 0u, v_mine = 0xffffffffu, n_mine = 0u;
  float c_mine = 0.f;
  double p_mine = 0.0;
  if (lane < count) {
    s_mine = perm[first + i0 + lane];
    c_mine = c[first + s_mine];
    v_mine = rec.vertex(first + s_mine);
    n_mine = min(rec.ord(first + s_mine), uint32_t(d.F - 1));
    // (z_mean given: `zhat` holds the product before its normalisation, which is applied here as the forward applied it)
    float zh = zhat[(long long)s_mine * d.F + n_mine];
    if (z_mean != nullptr) zh = (zh - z_mean[n_mine]) * z_rstd[n_mine];
    p_mine = double(c_mine) * double(zh);
  }
  // runs of equal vertices: bit l of `starts` says that entry l begins one
  const uint32_t v_before = uint32_t(__shfl_up(int(v_mine), 1, kWave));
  const unsigned long long starts = __ballot(lane < count && (lane == 0 || v_mine != v_before));
  const int quads = K / 4;
  auto lane_value = [&](uint32_t mine, int j) { return uint32_t(__builtin_amdgcn_readlane(int(mine), j)); };
  for (int q0 = 0; q0 < quads; q0 += kSegmentQuads * kWave) {
    unsigned long long left = starts;
    while (left) {
      const int a = __builtin_ctzll(left);
      left &= left - 1;
      const int b = left ? __builtin_ctzll(left) : count;  // the run is entries a .. b - 1
      const long long n = lane_value(n_mine, a);
      Vec4 acc[kSegmentQuads];
#pragma unroll
      for (int q = 0; q < kSegmentQuads; ++q) acc[q] = Vec4{0.f, 0.f, 0.f, 0.f};
      double m2 = 0.0;
      for (int j0 = a; j0 < b; j0 += kSegmentRows) {
        Vec4 xv[kSegmentRows][kSegmentQuads];
        float cj[kSegmentRows];
#pragma unroll
        for (int r = 0; r < kSegmentRows; ++r) {
          const int j = min(j0 + r, b - 1);  // (past the run's end: its last row again, weight 0)
          const float *row = xc + (long long)lane_value(s_mine, j) * K;
          cj[r] = j0 + r < b ? __uint_as_float(lane_value(__float_as_uint(c_mine), j)) : 0.f;
#pragma unroll
          for (int q = 0; q < kSegmentQuads; ++q) {
            const int col = q0 + q * kWave + lane;
            xv[r][q] = col < quads ? *reinterpret_cast<const Vec4 *>(row + 4 * col) : Vec4{0.f, 0.f, 0.f, 0.f};
          }
          if (q0 == 0 && j0 + r < b)
            m2 += __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(p_mine), j),
                                   __builtin_amdgcn_readlane(__double2loint(p_mine), j));
        }
#pragma unroll
        for (int r = 0; r < kSegmentRows; ++r)
#pragma unroll
          for (int q = 0; q < kSegmentQuads; ++q)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[q][e] += cj[r] * xv[r][q][e];
      }
#pragma unroll
      for (int q = 0; q < kSegmentQuads; ++q) {
        const int col = q0 + q * kWave + lane;
        if (col < quads) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (acc[q][e] != 0.f) atomicAdd(acc_out + n * K + 4 * col + e, acc[q][e]);
        }
      }
      if (q0 == 0 && lane == 0 && m2 != 0.0) atomicAdd(m2sum + n, m2);
    }
  }
}

// dlin[n, k] = rstd[n] * (sparse[n, k] - (m2sum[n] / B) * rstd[n] * dense[n, k])
__global__ __launch_bounds__(256) void combine_dlin_kernel(long long N, int K, double B, const float *__restrict__ sparse,
                                                           const float *__restrict__ dense,
                                                           const float *__restrict__ rstd,
                                                           const double *__restrict__ m2sum, float *__restrict__ dlin) {
  const long long quads = N * (K / 4);
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < quads; i += (long long)gridDim.x * 256) {
    const long long n = i / (K / 4);
    const float r = rstd[n], f = float(m2sum[n] / B) * r;
    const Vec4 a = *reinterpret_cast<const Vec4 *>(sparse + 4 * i), b = *reinterpret_cast<const Vec4 *>(dense + 4 * i);
    Vec4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = r * (a[e] - f * b[e]);
    *reinterpret_cast<Vec4 *>(dlin + 4 * i) = o;
  }
}

struct ProjectionForestLayout {
  size_t forest, colsum, m2sum, xc, gram, partials, dense, sparse, perm, total;
};

ProjectionForestLayout projection_forest_layout(const ForestDims &d, long long K) {
  ProjectionForestLayout l;
  size_t at = 0;
  auto take = [&](size_t bytes) {
    const size_t here = at;
    at += align_up(bytes, 256);
    return here;
  };
  l.forest = take(forest_backward_records_workspace<float>(d, HT_BACKWARD_ATOMIC, false, true, true));
  l.colsum = take(size_t(K) * sizeof(double));
  l.m2sum = take(size_t(d.F) * sizeof(double));
  l.xc = take(size_t(d.S) * K * sizeof(float));
  l.gram = take(size_t(K) * K * sizeof(float));
  const int shares = reduction_shares(K, K, d.S);
  l.partials = take(shares > 1 ? size_t(shares) * K * K * sizeof(float) : 0);
  l.dense = take(size_t(d.F) * K * sizeof(float));
  l.sparse = take(size_t(d.F) * K * sizeof(float));
  l.perm = take(size_t(d.T) * d.S * sizeof(uint32_t));
  l.total = at;
  return l;
}

template <bool COMPACT>
int projection_forest_sparse(const ForestDims &d, long long K, const void *records, const float *c, const float *xc,
                             const float *zhat, const float *z_mean, const float *z_rstd, uint32_t *perm, float *sparse,
                             double *m2sum, hipStream_t stream) {
  // (the records are only read here; c comes from the forest pass)
  const Records<float, COMPACT> rec = carve_records<float, COMPACT>(d, const_cast<void *>(records), nullptr);
  auto bucket = bucket_kernel<COMPACT>;
  hipLaunchKernelGGL(bucket, dim3((unsigned)d.T), dim3(kBucketThreads), size_t(d.V) * sizeof(uint32_t), stream, d, rec,
                     perm);
  HT_LAUNCH_CHECK("projection + forest backward (samples by vertex)");
  const long long waves = (long long)d.T * ((d.S + kWave - 1) / kWave);
  hipLaunchKernelGGL(segment_sums_kernel<COMPACT>, dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, stream, d, rec, c,
                     perm, xc, int(K), zhat, z_mean, z_rstd, sparse, m2sum);
  HT_LAUNCH_CHECK("projection + forest backward (segment sums)");
  return HT_OK;
}

}  // namespace

size_t projection_forest_forward_workspace(const ForestDims &d) {
  return align_up(projection_workspace(d.F), 256) + forest_forward_workspace<float>(d);
}

// The forward pass of the whole front: z [B x N] = x [B x K] * lin [N x K]^T with its batch statistics (mean, rstd, var
// [N] out), then the forest over the normalised product -- which is never written: the forest's kernels normalise z as
// they read it ((z - mean) * rstd, the arithmetic of bn_apply_kernel), one pass over [B x N] less than
// projection_forward + forest_forward. records (optional) as for forest_forward.
int projection_forest_forward(const ForestDims &d, bool fern, long long K, const float *x, const float *lin, double eps,
                              const float *thr, const int64_t *ord, const float *w, float *out, float *z, float *mean,
                              float *rstd, float *var, void *records, void *ws, size_t ws_bytes, hipStream_t stream) {
  int rc;
  if (d.K != 1) return fail(HT_ERR_INVALID_ARGUMENT, "Error: the projection's forest has no inner data dimensions.");
  if (ws == nullptr || ws_bytes < projection_forest_forward_workspace(d))
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: workspace too small for the forward pass.");
  const long long B = d.S, N = d.F;
  double *stats = static_cast<double *>(ws);
  if ((rc = zero_fill(stats, size_t(2) * N * sizeof(double), stream)) != HT_OK) return rc;
  if (B == 0 || N == 0) return HT_OK;
  if ((rc = launch_gemm<true, true, true>(x, K, lin, K, z, N, B, N, K, stats, stream)) != HT_OK) return rc;
  hipLaunchKernelGGL(bn_finalize_kernel, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, stream, stats, int(N), B, eps,
                     mean, rstd, var);
  HT_LAUNCH_CHECK("batch statistics");
  FeatureNorm<float> norm;
  norm.mean = mean, norm.rstd = rstd;
  unsigned char *forest_ws = static_cast<unsigned char *>(ws) + align_up(projection_workspace(N), 256);
  return forest_forward<float>(d, fern, z, thr, ord, w, out, records, forest_ws,
                               ws_bytes - align_up(projection_workspace(N), 256), stream, nullptr, &norm);
}

// Whether projection_forest_backward serves a forest [B x N features, K = 1] behind a projection from K_in inputs.
bool projection_forest_backward_ok(const ForestDims &d, long long K) {
  if (is_empty(d) || d.K != 1 || K <= 0 || K % 4 != 0 || d.V > kMaxBucketVertices) return false;
  if ((long long)d.T * d.V > 0x7fffffffLL * 4 || d.S > 0xffffffffLL) return false;
  return forest_backward_keeps_c<float>(d);
}

size_t projection_forest_backward_workspace(const ForestDims &d, long long K) {
  return projection_forest_backward_ok(d, K) ? projection_forest_layout(d, K).total : 0;
}

// dThr, dW of the forest and dLin of the projection in front of it, from the forest's walk records and upstream
// gradient gout; no dense dL/dzhat is formed. x [B x K], lin [N x K], zhat [B x N], rstd [N] as projection_forward left
// them -- or, with mean [N] given, `zhat` is the product before its normalisation as projection_forest_forward left it;
// dthr / dw / dlin may be null.
int projection_forest_backward(const ForestDims &d, bool fern, long long K, const float *x, const float *lin,
                               const float *zhat, const float *mean, const float *rstd, const float *w, const float *gout,
                               const void *records, float *dthr, float *dw, float *dlin, void *ws, size_t ws_bytes,
                               hipStream_t stream) {
  int rc;
  if (!projection_forest_backward_ok(d, K))
    return fail(HT_ERR_RUNTIME, "Error: this shape is not served by the records form of the projection backward.");
  const ProjectionForestLayout l = projection_forest_layout(d, K);
  if (ws == nullptr || ws_bytes < l.total)
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: workspace too small for the backward pass.");
  if (reinterpret_cast<uintptr_t>(x) % 16 != 0 || reinterpret_cast<uintptr_t>(lin) % 16 != 0 ||
      (dlin && reinterpret_cast<uintptr_t>(dlin) % 16 != 0) || reinterpret_cast<uintptr_t>(ws) % 16 != 0)
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: x, lin, dlin and the workspace must be 16-byte aligned.");
  unsigned char *base = static_cast<unsigned char *>(ws);
  const float *c = nullptr;
  const size_t forest_bytes = l.colsum - l.forest;
  if ((rc = forest_backward_records_keep_c<float>(d, fern, w, gout, records, dthr, dw, base + l.forest, forest_bytes,
                                                  stream, &c)) != HT_OK)
    return rc;
  if (!dlin) return HT_OK;
  const long long B = d.S, N = d.F;
  double *colsum = reinterpret_cast<double *>(base + l.colsum), *m2sum = reinterpret_cast<double *>(base + l.m2sum);
  float *xc = reinterpret_cast<float *>(base + l.xc), *gram = reinterpret_cast<float *>(base + l.gram);
  float *partials = reinterpret_cast<float *>(base + l.partials), *dense = reinterpret_cast<float *>(base + l.dense);
  float *sparse = reinterpret_cast<float *>(base + l.sparse);
  uint32_t *perm = reinterpret_cast<uint32_t *>(base + l.perm);
  // colsum and m2sum are neighbours: one clear
  if ((rc = zero_fill(colsum, l.xc - l.colsum, stream)) != HT_OK) return rc;
  if ((rc = zero_fill(sparse, size_t(N) * K * sizeof(float), stream)) != HT_OK) return rc;
  // (x is small beside the matrices of the forward pass: shares of 16 rows or more, enough of them to fill the device)
  const dim3 grid((unsigned)((K + 1023) / 1024), (unsigned)(B < 16 ? 1 : (B / 16 < 1024 ? B / 16 : 1024)));
  const dim3 sums_grid((unsigned)((K / 4 + kWave - 1) / kWave), (unsigned)(B < 64 ? 1 : (B / 64 < 256 ? B / 64 : 256)));
  hipLaunchKernelGGL(col_sums_kernel, sums_grid, dim3(256), 0, stream, x, B, int(K), colsum);
  HT_LAUNCH_CHECK("projection + forest backward (column means)");
  hipLaunchKernelGGL(center_kernel, grid, dim3(256), 0, stream, x, B, int(K), colsum, xc);
  HT_LAUNCH_CHECK("projection + forest backward (centring)");
  // Gc = xc^T xc (reduction over the batch, shares summed in a fixed order), dense = lin * Gc (Gc is symmetric: its
  // rows serve as the columns the product wants, reduction index contiguous)
  if ((rc = launch_gemm_batched<false, false, false, false>(xc, K, 0, xc, K, 0, gram, K, 0, K, K, B, 1, nullptr, nullptr,
                                                            nullptr, stream, false, partials,
                                                            reduction_shares(K, K, B), nullptr, true)) != HT_OK)
    return rc;
  if ((rc = launch_gemm<true, true, false>(lin, K, gram, K, dense, K, N, K, K, nullptr, stream)) != HT_OK) return rc;
  rc = compact_ok(d) ? projection_forest_sparse<true>(d, K, records, c, xc, zhat, mean, rstd, perm, sparse, m2sum, stream)
                     : projection_forest_sparse<false>(d, K, records, c, xc, zhat, mean, rstd, perm, sparse, m2sum, stream);
  if (rc != HT_OK) return rc;
  const long long quads = N * (K / 4);
  hipLaunchKernelGGL(combine_dlin_kernel, dim3((unsigned)((quads + 255) / 256 < 8192 ? (quads + 255) / 256 : 8192)),
                     dim3(256), 0, stream, N, int(K), double(B), sparse, dense, rstd, m2sum, dlin);
  HT_LAUNCH_CHECK("projection + forest backward (dLin)");
  return HT_OK;
}

// Linear mix over the tree axis behind a forest (the reference's "fused linear" operators,
// hingetree_fused_linear.cpp:75-412): f [B, T, R] are forest outputs (R = inner data positions x outputs per leaf).
//   forward : out[b, o, r] = bias[o] + sum_t lin[o, t] * f[b, t, r]
//   backward: h[b, t, r] = sum_o lin[o, t] * g[b, o, r]   (the upstream gradient of the forest)
//             dlin[o, t] = sum_{b, r} g[b, o, r] * f[b, t, r]
// rows [n][R] (the R values of a row contiguous) -> planes [R][n], and back. A thread takes a row: its R values are
// read (written) one after the other -- neighbouring threads' rows are neighbours in memory, so the lines are used
// whole -- and each plane is written (read) with consecutive threads on consecutive addresses.
__global__ __launch_bounds__(256) void rows_to_planes_kernel(long long n, int R, const float *__restrict__ rows,
                                                             float *__restrict__ planes) {
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256)
    for (int r = 0; r < R; ++r) planes[(long long)r * n + i] = rows[i * R + r];
}
__global__ __launch_bounds__(256) void planes_to_rows_kernel(long long n, int R, const float *__restrict__ planes,
                                                             float *__restrict__ rows) {
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256)
    for (int r = 0; r < R; ++r) rows[i * R + r] = planes[(long long)r * n + i];
}

int rows_to_planes(long long n, long long R, const float *rows, float *planes, bool back, hipStream_t stream) {
  if (n <= 0 || R <= 0) return HT_OK;
  if (R > 0x7fffffffLL) return fail(HT_ERR_RUNTIME, "Error: rows too long for this build.");
  long long blocks = (n + 255) / 256;
  if (blocks > 32 * kNumCUs) blocks = 32 * kNumCUs;
  if (back)
    hipLaunchKernelGGL(planes_to_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, n, int(R), rows, planes);
  else
    hipLaunchKernelGGL(rows_to_planes_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, n, int(R), rows, planes);
  HT_LAUNCH_CHECK("rows <-> planes");
  return HT_OK;
}

int mix_forward(long long B, long long T, long long O, long long R, const float *f, const float *lin,
                const float *bias, float *out, hipStream_t stream) {
  if (R == 1)  // out [B x O] = f [B x T] * lin [O x T]^T, bias per column
    return launch_gemm_batched<true, true, false, false>(f, T, 0, lin, T, 0, out, O, 0, B, O, T, 1, nullptr, nullptr, bias,
                                                         stream);
  // per sample: out_b [O x R] = lin [O x T] * f_b [T x R], bias per row
  return launch_gemm_batched<true, false, false, false>(lin, T, 0, f, R, T * R, out, R, O * R, O, R, T, B, nullptr, bias,
                                                        nullptr, stream);
}

// Area for the shares of the reproducible split of dLin's reduction (R == 1: one product reducing over the samples).
size_t mix_backward_workspace(long long B, long long T, long long O, long long R) {
  if (R != 1) return 0;
  const int shares = reduction_shares(O, T, B);
  return shares > 1 ? size_t(shares) * size_t(O) * size_t(T) * sizeof(float) : 0;
}

int mix_backward(long long B, long long T, long long O, long long R, const float *f, const float *lin, const float *g,
                 float *h, float *dlin, bool deterministic, hipStream_t stream, void *ws, size_t ws_bytes) {
  int rc;
  if (h) {
    if (R == 1)  // h [B x T] = g [B x O] * lin [O x T]
      rc = launch_gemm_batched<true, false, false, false>(g, O, 0, lin, T, 0, h, T, 0, B, T, O, 1, nullptr, nullptr,
                                                          nullptr, stream);
    else  // per sample: h_b [T x R] = lin^T [T x O] * g_b [O x R]
      rc = launch_gemm_batched<false, false, false, false>(lin, T, 0, g, R, O * R, h, R, T * R, T, R, O, B, nullptr,
                                                           nullptr, nullptr, stream);
    if (rc != HT_OK) return rc;
  }
  if (dlin && (B == 0 || R == 0)) return zero_fill(dlin, size_t(O) * size_t(T) * sizeof(float), stream);
  if (dlin) {
    if (R == 1) {  // dlin [O x T] = g^T [O x B] * f [B x T]
      // deterministic mode with a workspace: shares of the reduction summed in a fixed order instead of one long pass
      const bool ordered = deterministic && ws != nullptr && ws_bytes >= mix_backward_workspace(B, T, O, R);
      rc = launch_gemm_batched<false, false, false, false>(g, O, 0, f, T, 0, dlin, T, 0, O, T, B, 1, nullptr, nullptr,
                                                           nullptr, stream, !deterministic,
                                                           ordered ? static_cast<float *>(ws) : nullptr,
                                                           ordered ? reduction_shares(O, T, B) : 0);
    }
    else  // dlin [O x T] = sum_b g_b [O x R] * f_b [T x R]^T
      rc = launch_gemm_batched<true, true, false, true>(g, R, O * R, f, R, T * R, dlin, T, 0, O, T, R, B, nullptr,
                                                        nullptr, nullptr, stream, !deterministic);
    if (rc != HT_OK) return rc;
  }
  return HT_OK;
}

}  // namespace ht
