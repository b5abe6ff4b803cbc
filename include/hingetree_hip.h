/*
 * hingetree_hip.h -- C ABI of the MI355X (gfx950) hinge forest / hinge fern library (libhingetree_hip.so).
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream (passed as void*, 0 = the null stream).
 * Nothing here allocates device memory: outputs and scratch ("workspace") are supplied by the caller, whose size
 * requirement is answered by the matching *_workspace query. All kernels are enqueued on `stream` and the call
 * returns without synchronising. Tensors are dense, row-major, and must not alias.
 *
 * Return value: HT_OK, or an error code with a message retrievable through ht_last_error() (thread local).
 * HT_ERR_INVALID_ARGUMENT corresponds to the reference's std::invalid_argument (Python ValueError) and HT_ERR_RUNTIME
 * to its std::runtime_error (Python RuntimeError), hingetree_error.h:38-49.
 *
 * Shapes (reference notation, hingetree.cpp:87-135):
 *   x    [B, F, K]   real          K = product of trailing data dims
 *   thr  [T, V]      real          V = 2^depth - 1 (tree, heap order) or depth (fern)
 *   ord  [T, V]      int64         0 <= ord < F  (validated by the caller, see ht_ordinal_range)
 *   w    [T, L, M]   real          L = 2^depth, M = product of trailing weight dims
 *   out  [B, T, K, M]
 */
#ifndef HINGETREE_HIP_H
#define HINGETREE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { HT_OK = 0, HT_ERR_INVALID_ARGUMENT = 1, HT_ERR_RUNTIME = 2, HT_ERR_HIP = 3 };
enum { HT_F32 = 0, HT_F64 = 1 };
enum { HT_TREE = 0, HT_FERN = 1 };
/* backward accumulation modes */
enum { HT_BACKWARD_ATOMIC = 0, HT_BACKWARD_DETERMINISTIC = 1 };

typedef struct ht_forest_shape {
  int64_t B, F, K, T, depth, M;
  int32_t dtype; /* HT_F32 | HT_F64 */
  int32_t kind;  /* HT_TREE | HT_FERN */
} ht_forest_shape;

#define HT_MAX_CONV_DIMS 3
typedef struct ht_conv_shape {
  int64_t B, C, Cout, depth, M;
  int32_t dtype, kind;
  int32_t nd; /* 1, 2 or 3 spatial dims */
  int64_t size[HT_MAX_CONV_DIMS], kernel[HT_MAX_CONV_DIMS], stride[HT_MAX_CONV_DIMS], padding[HT_MAX_CONV_DIMS],
      dilation[HT_MAX_CONV_DIMS];
} ht_conv_shape;

/* Tile <-> image permutation (contract / expand): image [planes, size...] <-> tiles [planes, tiles..., window...]. */
typedef struct ht_tile_shape {
  int64_t planes;    /* batch * channels */
  int32_t nd;        /* 2 or 3 spatial dims */
  int32_t elem_size; /* 1, 2, 4 or 8 bytes: the elements are moved, never interpreted */
  int64_t size[3], tiles[3], window[3], padding[3];
} ht_tile_shape;

/* Message of the last failing call on this thread ("" if none). */
const char *ht_last_error(void);
/* ABI version of this header: bumped on any change of a signature or of a contract that a caller's buffers rest on
 * (what a workspace or records size covers, what a later call expects an earlier one to have written there).
 * ht_abi_version() returns the value the library was built with; a host compiled against this header compares it with
 * HT_ABI_VERSION and refuses a library built from another one. */
#define HT_ABI_VERSION 3
int ht_abi_version(void);
/* HT_OK if GPU `device` can run this library's code object (gfx950), else an error that names what it is. The tile
 * sizes assume that part's 160 KB of LDS per workgroup, 256 compute units and 8 L2 domains; hosts call this once per
 * device before the first launch. No counterpart in the reference, which compiles for whatever nvcc targets. */
int ht_check_device(int32_t device);

/* Device-side min and max of n int64 ordinals -> minmax[0], minmax[1] (device memory, 2 x int64).
 * Replaces the reference's per-call `inOrdinals.min()/.max()` range check (hingetree.cpp:91, hingetree_gpu.cu:445):
 * the caller reads the two values back and raises the reference's error. */
int ht_ordinal_range(const int64_t *ord, int64_t n, int64_t *minmax, void *stream);

/* out[b,t,k,m] = |margin| * w[t,leaf,m].
 * Replaces hingetree_gpu_forward / hingefern forward (hingetree.cpp:45,648-693; hingetree_gpu.cu:416-498). */
size_t ht_forest_forward_workspace(const ht_forest_shape *s);
int ht_forest_forward(const ht_forest_shape *s, const void *x, const void *thr, const int64_t *ord, const void *w,
                      void *out, void *workspace, size_t workspace_bytes, void *stream);

/* ht_forest_forward for callers that cannot allocate device memory -- code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc. No counterpart in the reference. Same result as ht_forest_forward, bit for
 * bit; the workspace (packed vertices, leaf rows at a line-friendly pitch) is an array of HT_STATIC_SCRATCH_BYTES bytes
 * inside the library's code object, one copy per GPU, held until the process ends. The call allocates and frees
 * nothing. A forest whose ht_forest_forward_workspace exceeds HT_STATIC_SCRATCH_BYTES is refused with
 * HT_ERR_INVALID_ARGUMENT (the headline forest -- 1000 trees of depth 10 with 10 outputs per leaf, 71 MB -- fits).
 * The first call on a device looks up that device's copy of the array; a call with an empty shape (B = 0) does only
 * that and launches nothing, so a caller can do it before a capture starts. All calls on one GPU share its array:
 * the kernels of a call rewrite what they read from it, so calls in stream order are independent of each other, and
 * calls that overlap on one GPU (different streams, different threads) race. */
#define HT_STATIC_SCRATCH_BYTES (80u << 20)
int ht_forest_forward_static(const ht_forest_shape *s, const void *x, const void *thr, const int64_t *ord,
                             const void *w, void *out, void *stream);

/* ht_forest_forward of a forest with inner data positions x [B, F, *tiles] and tile-shaped outputs per leaf
 * w [T, L, *window], whose result is stored directly as the image [B, T, *size] that ht_expand makes of
 * [B, T, *tiles, *window] (g: planes = B * T, elem_size = that of the data type; image positions no tile covers are 0).
 * One call in place of the pair hingetree_gpu_forward (hingetree_gpu.cu:416-498) + expand_gpu (expand_gpu.cu:110-172)
 * that the reference's segmentation model runs back to back (rcc/Net.py:99-109): the [B, T, *tiles, *window]
 * intermediate is never written. Same workspace as ht_forest_forward. */
int ht_forest_forward_image(const ht_forest_shape *s, const ht_tile_shape *g, const void *x, const void *thr,
                            const int64_t *ord, const void *w, void *image, void *workspace, size_t workspace_bytes,
                            void *stream);

/* Gradients of the above w.r.t. x, thr and w; any of dx/dthr/dw may be NULL (not requested). The library clears the
 * requested buffers itself and then accumulates into them.
 * mode HT_BACKWARD_ATOMIC replaces hingetree_gpu_backward (hingetree.cpp:48,695-740; hingetree_gpu.cu:619-730);
 * mode HT_BACKWARD_DETERMINISTIC replaces hingetree_gpu_backward_deterministic (hingetree.cpp:51,742-787;
 * hingetree_gpu.cu:500-617) and is bit-reproducible run to run. */
size_t ht_forest_backward_workspace(const ht_forest_shape *s, int mode, int need_dx, int need_dthr, int need_dw);
int ht_forest_backward(const ht_forest_shape *s, const void *x, const void *thr, const int64_t *ord, const void *w,
                       const void *gout, void *dx, void *dthr, void *dw, int mode, void *workspace,
                       size_t workspace_bytes, void *stream);

/* ht_forest_backward whose upstream gradient is still the image [B, T, *size] (the gradient of what
 * ht_forest_forward_image stored): one call in place of the pair contract2d_gpu / contract3d_gpu (expand_gpu.cu:110-151,
 * 198-295, reached through _Expand.backward, _HingeTree.py:54-60) + hingetree_gpu_backward (hingetree_gpu.cu:619-730) -- the tile-major
 * [B, T, *tiles, *window] gradient is never written; image positions outside the tiles are not read. Same workspace
 * as ht_forest_backward. Served for float32 data in atomic mode with 16 to 256 outputs per leaf (four times a power of
 * two) whose innermost window, padding and image extents are multiples of four; ht_forest_backward_image_supported
 * returns 1 for those and 0 otherwise (contract the gradient and call ht_forest_backward then), and
 * ht_forest_backward_image fails with HT_ERR_INVALID_ARGUMENT where it would return 0. */
int ht_forest_backward_image_supported(const ht_forest_shape *s, const ht_tile_shape *g, int mode, int need_dx,
                                       int need_dthr, int need_dw);
int ht_forest_backward_image(const ht_forest_shape *s, const ht_tile_shape *g, const void *x, const void *thr,
                             const int64_t *ord, const void *w, const void *gout_image, void *dx, void *dthr, void *dw,
                             int mode, void *workspace, size_t workspace_bytes, void *stream);

/* Training path, no counterpart in the reference (whose backward walks every tree again, hingetree_gpu.cu:619-730):
 * ht_forest_forward_records is ht_forest_forward that also writes what its walks found -- leaf key, selected vertex,
 * its ordinal and the signed margin of every (tree, sample) pair -- into `records`, an opaque device buffer of
 * ht_forest_records_bytes(s) bytes that the caller keeps until the matching ht_forest_backward_records call, which
 * computes the same gradients as ht_forest_backward from w, the upstream gradient and the records alone (x, thr and ord
 * are not read again). ht_forest_records_bytes returns 0 for shapes the records path does not serve (use the stateless
 * pair then). The records are only valid for the x / thr / ord of the forward call that wrote them. */
size_t ht_forest_records_bytes(const ht_forest_shape *s);
int ht_forest_forward_records(const ht_forest_shape *s, const void *x, const void *thr, const int64_t *ord,
                              const void *w, void *out, void *records, size_t records_bytes, void *workspace,
                              size_t workspace_bytes, void *stream);
size_t ht_forest_backward_records_workspace(const ht_forest_shape *s, int mode, int need_dx, int need_dthr,
                                            int need_dw);
int ht_forest_backward_records(const ht_forest_shape *s, const void *w, const void *gout, const void *records,
                               size_t records_bytes, void *dx, void *dthr, void *dw, int mode, void *workspace,
                               size_t workspace_bytes, void *stream);

/* Per-(b,t,k) leaf key / signed margin + selected ordinal / per-(t,leaf) visit counts; any output may be NULL.
 * Replaces hingetree_gpu_leafmap, _marginmap, _reachability (hingetree.cpp:54-60; hingetree_gpu.cu:732-933), which
 * return the leaf map and the counts as int64 on the GPU. The workspace (its size depends on whether `reach` will be
 * asked for) holds the packed vertices that let the maps run on the forward pass's walk and, for `reach`, 16-bit leaf
 * keys for a histogram per tree; the call works without it or with less -- maps several times slower, counts from one
 * global atomic per pair. */
size_t ht_forest_maps_workspace(const ht_forest_shape *s, int32_t want_reach);
int ht_forest_maps(const ht_forest_shape *s, const void *x, const void *thr, const int64_t *ord, int64_t *leafmap,
                   void *margins, int64_t *ordinals, int64_t *reach, void *workspace, size_t workspace_bytes,
                   void *stream);

/* Convolutional variant, groups == 1: one tree per (out channel, in channel) over the prod(kernel) taps of that in
 * channel's patch, summed over in channels; the patch gather happens inside the walk (no im2col buffer).
 *   x [B, C, *size]   thr/ord [Cout, C, V]   w [Cout, C, L, M]   out [B, Cout, *out_size, M]
 * Replaces hingetree_conv_gpu_forward / _backward (hingetree_conv.cpp:31-47; hingetree_conv_gpu.cu:214-618) and the
 * ImageToMatrix extraction kernels they launch (ImageToMatrix_gpu.cu:132-239). */
int ht_conv_output_size(const ht_conv_shape *s, int64_t *out_size /* [nd] */);
int ht_conv_forward(const ht_conv_shape *s, const void *x, const void *thr, const int64_t *ord, const void *w, void *out,
                    void *stream);
int ht_conv_backward(const ht_conv_shape *s, const void *x, const void *thr, const int64_t *ord, const void *w,
                     const void *gout, void *dx, void *dthr, void *dw, void *stream);

/* ---- dense projection + batch normalisation in front of a forest (fp32) --------------------------------------------
 * The reference has no operator for this stage: its README and experiments compose torch.nn.Linear(bias=False),
 * torch.nn.BatchNorm1d(affine=False) and RandomHingeForest (README.md:117-129, experiments/run_letter_seq.py:45-52).
 * These two calls replace the first two modules of that composition in training mode; the forest operators above
 * consume zhat unchanged.
 *   forward : zhat [B, N] = (z - mean) * rstd with z = x [B, K] * lin [N, K]^T computed on the matrix cores; the batch
 *             sums of z are accumulated by the same kernel. mean, rstd, var [N] are outputs (var: biased variance, for
 *             the caller's running statistics; may be NULL).
 *   backward: g [B, N] holds dL/dzhat on entry; dlin [N, K] and dx [B, K] receive the parameter / input gradients
 *             (either may be NULL). With dx, g is overwritten with dL/dz; without it g is left as it came (the
 *             normalisation's backward is then applied while the dlin product loads g, with the same result).
 * workspace: ht_projection_workspace(N) bytes for the forward pass, ht_projection_backward_workspace(B, K, N) for the
 * backward pass (a small layer under a large batch splits the batch reduction of dlin over workgroups and sums their
 * shares in a fixed order, so the result does not depend on scheduling). */
size_t ht_projection_workspace(int64_t N);
size_t ht_projection_backward_workspace(int64_t B, int64_t K, int64_t N);
int ht_projection_forward(int64_t B, int64_t K, int64_t N, const float *x, const float *lin, double eps, float *zhat,
                          float *mean, float *rstd, float *var, void *workspace, size_t workspace_bytes, void *stream);
int ht_projection_backward(int64_t B, int64_t K, int64_t N, const float *x, const float *lin, const float *zhat,
                           const float *rstd, float *g, float *dlin, float *dx, void *workspace,
                           size_t workspace_bytes, void *stream);

/* The backward pass of the whole front -- Linear(bias = False) -> BatchNorm1d(affine = False) -> forest in training
 * mode -- from the walk records of ht_forest_forward_records run on zhat: dthr [T, V], dw [T, L, M] of the forest and
 * dlin [N, K_in] of the projection (each may be NULL), for a caller that wants no gradient of the projection's input.
 * No counterpart in the reference, whose composition multiplies a dense dL/dzhat [B, N] by the inputs; here that
 * matrix is never formed: it holds one non-zero per (sample, tree), so
 *   dlin[n, :] = rstd[n] * (sum over the pairs that selected feature n of c * xc[sample, :]
 *                           - mean_b(g * zhat)[n] * rstd[n] * (lin * xc^T xc)[n, :]),   xc = x - mean_b x,
 * with c the forest's input gradient at the selected vertex: a sparse sum over the records plus two small dense
 * products, which agrees with the dense form to rounding (sums reordered, nothing cancelled).
 *   forest: the forest's shape with B = batch, F = N (the projected features), K = 1, dtype HT_F32; x [B, K_in],
 *   lin [N, K_in], zhat [B, N], rstd [N] as ht_projection_forward took / left them; w, gout, records as for
 *   ht_forest_backward_records. Atomic accumulation (the order of additions, hence the last bits, can differ between
 *   runs). ht_projection_forest_backward_workspace returns 0 where the shape is not served (K_in not a multiple of 4,
 *   K > 1, more than 16384 vertices per tree, shapes whose records the staged kernels do not take): call
 *   ht_forest_backward_records + ht_projection_backward there.
 *   mean [N]: NULL when `zhat` is the normalised product; when `zhat` is the product z before its normalisation, as
 *   ht_projection_forest_forward leaves it, its batch means (the normalisation is then applied where zhat is read).
 * ht_projection_forest_forward is the matching forward pass: z [B, N] = x * lin^T on the matrix cores with its batch
 * statistics (mean, rstd [N]; var [N], biased, may be NULL), then the forest over (z - mean) * rstd, which is not
 * written out -- the forest's kernels normalise z as they read it, with the two rounded operations a separate pass
 * would use, so `out` equals that of ht_projection_forward + ht_forest_forward_records bit for bit and the records hold
 * the same walks.
 * records may be NULL (no backward pass will follow). */
size_t ht_projection_forest_forward_workspace(const ht_forest_shape *forest);
int ht_projection_forest_forward(const ht_forest_shape *forest, int64_t K_in, const float *x, const float *lin, double eps,
                                 const float *thr, const int64_t *ord, const float *w, float *out, float *z, float *mean,
                                 float *rstd, float *var, void *records, size_t records_bytes, void *workspace,
                                 size_t workspace_bytes, void *stream);
size_t ht_projection_forest_backward_workspace(const ht_forest_shape *forest, int64_t K_in);
int ht_projection_forest_backward(const ht_forest_shape *forest, int64_t K_in, const float *x, const float *lin,
                                  const float *zhat, const float *mean, const float *rstd, const float *w, const float *gout,
                                  const void *records, size_t records_bytes, float *dthr, float *dw, float *dlin,
                                  void *workspace, size_t workspace_bytes, void *stream);

/* Diagnostic, host only, no counterpart in the reference: the matrix-product kernel's launch-slot -> result-tile map
 * for a grid of tiles_i x tiles_j result tiles (slots are dealt to the 8 L2 domains round robin; each domain walks a
 * band of tile rows in panels of 8 tile columns). tile_i / tile_j receive one entry per launch slot, (-1, -1) for a
 * slot that has no tile; ((tiles_i + 7) / 8) * tiles_j * 8 slots exist and `capacity` entries must be available.
 * Exists so that a host-side test can check that every tile is computed exactly once. */
int ht_gemm_tile_map(int32_t tiles_i, int32_t tiles_j, int32_t *tile_i, int32_t *tile_j, int64_t capacity);

/* ---- linear mix over the tree axis behind a forest (fp32) ------------------------------------------------------------
 * The dense half of the reference's fused-linear operators tree_fused_linear_forward / _backward and fern_*
 * (hingetree_fused_linear.cpp:75-412; GPU: hingetree_fused_linear_gpu.cu, which accumulates the forward with global
 * atomics). The forest half is ht_forest_forward / ht_forest_backward above; f [B, T, R] is the forest's output with
 * R = K * M (inner data positions x outputs per leaf).
 *   forward : out [B, O, R] = bias[o] + sum_t lin[o, t] * f[b, t, r]           (bias may be NULL)
 *   backward: h [B, T, R]   = sum_o lin[o, t] * g[b, o, r]   -> upstream gradient for ht_forest_backward (may be NULL)
 *             dlin [O, T]   = sum_{b, r} g[b, o, r] * f[b, t, r]                (may be NULL)
 * Both run on the matrix cores. The forward and h use no atomics. dlin of a narrow head has few result tiles and a
 * long reduction: unless `deterministic` is set its reduction is split over workgroups whose shares meet in float
 * atomics (an order of magnitude faster, not bit-reproducible run to run). */
int ht_tree_mix_forward(int64_t B, int64_t T, int64_t O, int64_t R, const float *f, const float *lin,
                        const float *bias, float *out, void *stream);
int ht_tree_mix_backward(int64_t B, int64_t T, int64_t O, int64_t R, const float *f, const float *lin, const float *g,
                         float *h, float *dlin, int deterministic, void *stream);

/* ht_tree_mix_backward with a workspace (ht_tree_mix_backward_workspace bytes; may be NULL / 0): in deterministic
 * mode the reduction of dlin over the samples (R == 1) is then split over workgroups whose shares are summed in a
 * fixed order, instead of running as one long reproducible pass. No counterpart in the reference. */
size_t ht_tree_mix_backward_workspace(int64_t B, int64_t T, int64_t O, int64_t R);
int ht_tree_mix_backward_ws(int64_t B, int64_t T, int64_t O, int64_t R, const float *f, const float *lin, const float *g,
                            float *h, float *dlin, int deterministic, void *workspace, size_t workspace_bytes,
                            void *stream);

/* Helpers for the mix with a few values per (sample, tree) (R = 2 ... ~100: extra outputs of a tabular forest), no
 * counterpart in the reference: rows [n][R] <-> planes [R][n]. With f, g, out and h moved to planes, the R slices are
 * R times as many samples of an R = 1 problem, and ht_tree_mix_forward / _backward serve them as ONE product with
 * B * R rows instead of B products whose results fill a sliver of a matrix-core tile each. */
int ht_rows_to_planes(int64_t n, int64_t R, const float *rows, float *planes, void *stream);
int ht_planes_to_rows(int64_t n, int64_t R, const float *planes, float *rows, void *stream);

/* The same three products for float64 data (the reference instantiates its fused-linear operators for double as well,
 * hingetree_fused_linear.cpp:798-806,845-853): plain kernels with a fixed summation order, always reproducible. */
int ht_tree_mix_forward_f64(int64_t B, int64_t T, int64_t O, int64_t R, const double *f, const double *lin,
                            const double *bias, double *out, void *stream);
int ht_tree_mix_backward_f64(int64_t B, int64_t T, int64_t O, int64_t R, const double *f, const double *lin,
                             const double *g, double *h, double *dlin, void *stream);

/* ---- contract / expand -----------------------------------------------------------------------------------------------
 * Replace contract2d/3d and expand2d/3d of the reference (expand.cpp:37-227 on the CPU, expand_gpu.cu:110-172 on the
 * GPU; exported as `contract` / `expand`, hingetree.cpp:2029-2030). Tile j of a dimension covers image positions
 * [j * window - padding, j * window - padding + window); what lies outside the image (contract) or is covered by no
 * tile (expand) is 0. Every element of `out` is written. */
int ht_contract(const ht_tile_shape *s, const void *image, void *tiles, void *stream);
int ht_expand(const ht_tile_shape *s, const void *tiles, void *image, void *stream);

/* Host-side (CPU pointers) threshold consistency, in place for _fix. One flag byte per tree is written to `flags`
 * (check: 1 = consistent; fix: 1 = changed). Ferns are always consistent and never change.
 * Replaces hingetree_cpu_check_thresholds / _fix_thresholds (hingetree.cpp:513-581, HingeTreeCommon.h:211-287); the
 * reference keeps these on the CPU as well (hingetree.cpp:936,1010). */
int ht_check_thresholds(const void *thr, const int64_t *ord, int64_t T, int64_t depth, int32_t dtype, int32_t kind,
                        uint8_t *flags);
int ht_fix_thresholds(void *thr, const int64_t *ord, int64_t T, int64_t depth, int32_t dtype, int32_t kind,
                      uint8_t *flags);

#ifdef __cplusplus
}
#endif
#endif /* HINGETREE_HIP_H */
