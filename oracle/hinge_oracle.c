/*
 * CPU oracle for the hinge forest / hinge fern forward + backward path.
 *
 * THIS IS TEST INFRASTRUCTURE. It restates, in plain single-threaded C, what the reference's CPU back-end computes
 * (hingetree.cpp, hingetree_conv.cpp, HingeTreeCommon.h, ImageToMatrix.h of NIH-MIP/HingeTreeForTorch) so that the
 * HIP kernels can be checked against it on machines where the reference itself is absent. Only tests, the smoke
 * check and the benchmark's CPU-baseline leg may load this library; the product never does.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   walk/forward/backward/maps, conv forward/backward, check/fix thresholds
 *       - bit-for-bit against the reference's own CPU sources compiled in place (oracle/_ref, when present)
 *       - against the committed vectors under tests/golden/ that were written from that build
 *       - against closed forms and a brute-force numpy restatement (depth-1 closed form, infinite thresholds,
 *         fern == tree with level-constant vertices, finite differences, dX/dThr conservation, F.unfold for conv)
 *   conv index matrix
 *       - against the 3-channel 6x5 / 3x4 kernel / pad 1 layout documented in ImageToMatrix.cpp:49-60 and F.unfold
 *
 * Built with -O2 -ffp-contract=off and no -march, like the reference's setup.py (-O2): no fused multiply-add, so
 * every product and sum rounds exactly where the reference's does.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ImageToMatrix.h:159-209 (validity + output size) and :304-333 (index matrix of ONE channel).
 * geom = { nd, size[nd], kernel[nd], stride[nd], pad[nd], dil[nd] }.
 * Returns a malloc'ed [rows, P] matrix: entry (p, j) is the flat offset inside one channel image of tap j of output
 * position p, or -1 when that tap lies in the padding. Output positions and taps are both enumerated in raster
 * order (last dimension fastest). NULL if the geometry is invalid. */
int64_t *ho_conv_index_matrix(const int64_t *geom, int64_t *rows_out, int64_t *taps_out, int64_t *in_count_out) {
  const int64_t nd = geom[0];
  if (nd < 1 || nd > 3) return NULL;
  const int64_t *size = geom + 1, *ker = size + nd, *str = ker + nd, *pad = str + nd, *dil = pad + nd;
  int64_t osz[3], rows = 1, taps = 1, in_count = 1;
  for (int64_t d = 0; d < nd; ++d) {
    if (ker[d] <= 0 || str[d] <= 0 || dil[d] <= 0 || pad[d] < 0 || size[d] < 1) return NULL;
    const int64_t win = ker[d] + (ker[d] - 1) * (dil[d] - 1);
    if (size[d] + 2 * pad[d] < win) return NULL;
    osz[d] = (size[d] + 2 * pad[d] - win) / str[d] + 1;
    rows *= osz[d]; taps *= ker[d]; in_count *= size[d];
  }
  int64_t *index = (int64_t *)malloc(sizeof(int64_t) * (size_t)(rows * taps));
  if (!index) return NULL;
  int64_t oc[3] = {0, 0, 0};
  for (int64_t p = 0; p < rows; ++p) {
    int64_t kc[3] = {0, 0, 0};
    for (int64_t j = 0; j < taps; ++j) {
      int64_t flat = 0, inside = 1;
      for (int64_t d = 0; d < nd; ++d) {
        const int64_t at = oc[d] * str[d] - pad[d] + kc[d] * dil[d];
        if (at < 0 || at >= size[d]) { inside = 0; break; }
        flat = flat * size[d] + at;
      }
      index[p * taps + j] = inside ? flat : -1;
      for (int64_t d = nd - 1; d >= 0; --d) { if (++kc[d] < ker[d]) break; kc[d] = 0; }
    }
    for (int64_t d = nd - 1; d >= 0; --d) { if (++oc[d] < osz[d]) break; oc[d] = 0; }
  }
  *rows_out = rows; *taps_out = taps; *in_count_out = in_count;
  return index;
}

/* Copies the index matrix into caller memory (for tests). Returns rows*taps, or -1 on invalid geometry; with
 * dst == NULL only the size is returned. */
int64_t ho_conv_index_matrix_copy(const int64_t *geom, int64_t *dst) {
  int64_t rows, taps, in_count;
  int64_t *index = ho_conv_index_matrix(geom, &rows, &taps, &in_count);
  if (!index) return -1;
  if (dst) memcpy(dst, index, sizeof(int64_t) * (size_t)(rows * taps));
  free(index);
  return rows * taps;
}

#define REAL float
#define FN(name) name##_f32
#define RABS fabsf
#include "hinge_oracle_impl.inc"
#undef REAL
#undef FN
#undef RABS

#define REAL double
#define FN(name) name##_f64
#define RABS fabs
#include "hinge_oracle_impl.inc"
#undef REAL
#undef FN
#undef RABS
