// Contract / Expand: the tile <-> image permutation that sits between a forest with tile-shaped extra outputs and an
// image-shaped loss in the reference's segmentation models (expand.cpp:37-227, expand_gpu.cu:110-172; used as
// extra_outputs = [8, 8] followed by Expand in rcc/Net.py:99-109).
//
//   contract: image [planes, size...] -> tiles [planes, tiles..., window...]; tile j of a dimension covers image
//             positions [j * window - padding, j * window - padding + window); positions outside the image read 0.
//   expand:   the inverse gather; image positions that no tile covers read 0.
// Both are written as gathers over the OUTPUT (every output element is written exactly once, so no clearing pass is
// needed) and move opaque elements of 1, 2, 4 or 8 bytes, which covers every dtype the reference accepts.
#include "common.hpp"

namespace ht {
namespace {

struct TileGeom {
  long long planes;
  int size[3], tiles[3], win[3], pad[3];
};

// 16 opaque bytes: where the innermost window extent, padding and image extent are all whole multiples of 16 bytes, a
// run of that many consecutive innermost elements is consecutive in both layouts and lies wholly inside or wholly
// outside, so the permutation can move such runs as single elements of a geometry with the innermost extents divided.
struct alignas(16) Word16 {
  uint32_t w[4];
};

template <typename Word, bool EXPAND>
__global__ __launch_bounds__(256) void tile_permute_kernel(TileGeom g, const Word *__restrict__ in,
                                                           Word *__restrict__ out, long long total) {
  const long long image = (long long)g.size[0] * g.size[1] * g.size[2];
  const long long wsz = (long long)g.win[0] * g.win[1] * g.win[2];
  const long long tiled = (long long)g.tiles[0] * g.tiles[1] * g.tiles[2] * wsz;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long long)gridDim.x * 256) {
    Word v = Word{};
    if (EXPAND) {
      const long long plane = i / image;
      long long r = i - plane * image;
      int p[3];
      p[2] = int(r % g.size[2]);
      r /= g.size[2];
      p[1] = int(r % g.size[1]);
      p[0] = int(r / g.size[1]);
      long long tile = 0, within = 0;
      bool covered = true;
#pragma unroll
      for (int dd = 0; dd < 3; ++dd) {
        const int q = p[dd] + g.pad[dd];
        const int j = q / g.win[dd], w = q - j * g.win[dd];
        covered = covered && j < g.tiles[dd];
        tile = tile * g.tiles[dd] + j;
        within = within * g.win[dd] + w;
      }
      if (covered) v = in[plane * tiled + tile * wsz + within];
    } else {
      const long long plane = i / tiled;
      long long r = i - plane * tiled;
      int w[3], j[3];
      for (int dd = 2; dd >= 0; --dd) {
        w[dd] = int(r % g.win[dd]);
        r /= g.win[dd];
      }
      for (int dd = 2; dd >= 0; --dd) {
        j[dd] = int(r % g.tiles[dd]);
        r /= g.tiles[dd];
      }
      long long at = 0;
      bool inside = true;
#pragma unroll
      for (int dd = 0; dd < 3; ++dd) {
        const int p = j[dd] * g.win[dd] - g.pad[dd] + w[dd];
        inside = inside && p >= 0 && p < g.size[dd];
        at = at * g.size[dd] + p;
      }
      if (inside) v = in[plane * image + at];
    }
    out[i] = v;
  }
}

template <bool EXPAND>
int launch_permute(const TileGeom &g, int elem_size, const void *in, void *out, hipStream_t stream) {
  const long long image = (long long)g.size[0] * g.size[1] * g.size[2];
  const long long tiled = (long long)g.tiles[0] * g.tiles[1] * g.tiles[2] * g.win[0] * g.win[1] * g.win[2];
  long long total = g.planes * (EXPAND ? image : tiled);
  if (total <= 0) return HT_OK;
  const int per16 = 16 / elem_size;  // elements in 16 bytes
  if (per16 > 1 && g.size[2] % per16 == 0 && g.win[2] % per16 == 0 && g.pad[2] % per16 == 0 &&
      reinterpret_cast<uintptr_t>(in) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0) {
    TileGeom wide = g;
    wide.size[2] /= per16;
    wide.win[2] /= per16;
    wide.pad[2] /= per16;
    total /= per16;
    long long blocks = (total + 255) / 256;
    if (blocks > 64 * kNumCUs) blocks = 64 * kNumCUs;
    hipLaunchKernelGGL((tile_permute_kernel<Word16, EXPAND>), dim3((unsigned)blocks), dim3(256), 0, stream, wide,
                       static_cast<const Word16 *>(in), static_cast<Word16 *>(out), total);
    HT_LAUNCH_CHECK((EXPAND ? "expand (16-byte runs)" : "contract (16-byte runs)"));
    return HT_OK;
  }
  long long blocks = (total + 255) / 256;
  if (blocks > 64 * kNumCUs) blocks = 64 * kNumCUs;
#define HT_PERMUTE(Word)                                                                                        \
  hipLaunchKernelGGL((tile_permute_kernel<Word, EXPAND>), dim3((unsigned)blocks), dim3(256), 0, stream, g,      \
                     static_cast<const Word *>(in), static_cast<Word *>(out), total)
  switch (elem_size) {
    case 1: HT_PERMUTE(uint8_t); break;
    case 2: HT_PERMUTE(uint16_t); break;
    case 4: HT_PERMUTE(uint32_t); break;
    case 8: HT_PERMUTE(unsigned long long); break;
    default: return fail(HT_ERR_INVALID_ARGUMENT, "Error: unsupported element size.");
  }
#undef HT_PERMUTE
  HT_LAUNCH_CHECK((EXPAND ? "expand" : "contract"));
  return HT_OK;
}

int make_tile_geom(const ht_tile_shape *s, TileGeom *g) {
  if (!s) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null shape.");
  if (s->nd != 2 && s->nd != 3)
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: Only 2D and 3D window sizes are supported.");
  if (s->planes < 0) return fail(HT_ERR_INVALID_ARGUMENT, "Error: negative tensor size.");
  g->planes = s->planes;
  const int shift = 3 - s->nd;  // a 2-d problem is a 3-d one with a leading dimension of extent 1
  for (int dd = 0; dd < 3; ++dd) {
    g->size[dd] = g->tiles[dd] = g->win[dd] = 1;
    g->pad[dd] = 0;
  }
  long long image = 1, tiled = 1;
  for (int dd = 0; dd < s->nd; ++dd) {
    if (s->size[dd] < 0 || s->tiles[dd] < 0 || s->window[dd] < 1 || s->padding[dd] < 0 ||
        s->size[dd] > 0x3fffffff || s->tiles[dd] > 0x3fffffff || s->window[dd] > 0x3fffffff ||
        s->padding[dd] > 0x3fffffff)
      return fail(HT_ERR_INVALID_ARGUMENT, "Error: invalid tile geometry.");
    g->size[dd + shift] = int(s->size[dd]);
    g->tiles[dd + shift] = int(s->tiles[dd]);
    g->win[dd + shift] = int(s->window[dd]);
    g->pad[dd + shift] = int(s->padding[dd]);
    image *= s->size[dd];
    tiled *= s->tiles[dd] * s->window[dd];
  }
  if (image > (1ll << 40) || tiled > (1ll << 40))
    return fail(HT_ERR_RUNTIME, "Error: image too large for this build.");
  return HT_OK;
}

}  // namespace

int tile_contract(const ht_tile_shape *s, const void *in, void *out, hipStream_t stream) {
  TileGeom g;
  int rc = make_tile_geom(s, &g);
  if (rc != HT_OK) return rc;
  return launch_permute<false>(g, s->elem_size, in, out, stream);
}

int tile_expand(const ht_tile_shape *s, const void *in, void *out, hipStream_t stream) {
  TileGeom g;
  int rc = make_tile_geom(s, &g);
  if (rc != HT_OK) return rc;
  return launch_permute<true>(g, s->elem_size, in, out, stream);
}

}  // namespace ht
