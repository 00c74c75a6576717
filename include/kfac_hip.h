/* kfac_hip.h -- C ABI of libkfac_hip.so: the K-FAC per-layer hot path of
 * tyohei/chainerkfac as hand-written HIP kernels for gfx950 (MI355X).
 *
 * Conventions
 *   - every entry point is extern "C", returns 0 on success and a negative
 *     KFAC_E* code on failure; kfac_last_error_string() describes the last
 *     failure of the calling thread.  Nothing throws.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).
 *     All work is enqueued on it; calls return without waiting for the GPU
 *     unless stated otherwise.
 *   - pointers named *_dev / x / gy / A / G / F / buf ... are device pointers
 *     that the library borrows for the duration of the enqueued work.  Tables
 *     (`ptrs`, `dims`, ...) are host arrays read before the call returns.
 *   - all matrices are float32, C-contiguous, row-major; Kronecker factors are
 *     full symmetric d x d arrays, as in the reference.
 *   - the library is thread-compatible: one thread per plan / stream at a time.
 *
 * Each entry point cites the reference code it replaces (paths relative to the
 * chainerkfac checkout).
 */
#ifndef KFAC_HIP_H_
#define KFAC_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KFAC_ABI_VERSION 1

#define KFAC_OK 0
#define KFAC_EINVAL (-1)   /* bad argument (shape, null pointer, size)        */
#define KFAC_EHIP (-2)     /* a HIP runtime call failed                        */
#define KFAC_ENOMEM (-3)   /* caller workspace too small / allocation failed   */

int kfac_abi_version(void);
const char *kfac_last_error_string(void);

/* Tuning options (no counterpart in the reference, which has no tunables on this
 * path).  Every option has a built-in default that the library chooses itself;
 * kfac_option_set overrides it for plans created and calls made afterwards,
 * kfac_option_unset restores the default.  The environment variable
 * KFAC_<NAME IN CAPITALS> gives an option its starting value; the environment is
 * read once, when the first option is looked up.  Names (kfac_option_name(i) for
 * i < kfac_option_count()):
 *   syrk_bm64_max, syrk_splits, conv_rows, rows_wm, shift_slices5, shift_slices3,
 *   conv_shift, conv_shift_strict, group_bm64_max, group_macro, group_panels,
 *   group_macro_tasks, group_graded, group_side_stream, inverse_group, inverse_border,
 *   inverse_lookahead, inverse_rest_lds, inverse_align, precond_tasks,
 *   bn_stats_loop, host_only (1: no call reaches the GPU -- plans are built and
 *   every entry point checks its arguments and walks its launch sites, for runs
 *   of the host code under a sanitizer on a machine without a GPU).
 * Not thread-safe against concurrent calls into the library. */
int kfac_option_set(const char *name, double value);
int kfac_option_unset(const char *name);
int kfac_option_get(const char *name, double *value, int *is_set);
int kfac_option_count(void);
const char *kfac_option_name(int index);

/* ------------------------------------------------------------------------
 * (4) Communicator buffer layout: triangular pack / unpack
 * --------------------------------------------------------------------- */

/* Packed length of a list of arrays: n(n+1)/2 for a triangular array of side
 * n = triangle_size[i] (> 0), sizes[i] otherwise.
 * Replaces communicators/_utility.py:72-83 (get_nelems).  Returns -1 on a
 * triangular entry whose size is not triangle_size^2. */
int64_t kfac_packed_nelems(int n_arrays, const int64_t *sizes,
                           const int32_t *triangle_size);

/* Descriptor of a list of arrays in buffer order; replaces _ArraysInfo
 * (communicators/pure_nccl_communicator.py:221-279).  The tables are uploaded
 * once; kfac_pack_plan_set_ptrs re-uploads only the pointers, and only when
 * they differ from the last ones: the upload is a copy ordered on `stream`, so
 * the pack / unpack calls that are to see it must be issued on that stream (or
 * on one that waits for it). */
typedef struct kfac_pack_plan *kfac_pack_plan_t;

int kfac_pack_plan_create(int n_arrays, const void *const *ptrs,
                          const int64_t *sizes, const int32_t *triangle_size,
                          const int32_t *rank_of, kfac_pack_plan_t *plan_out);
int kfac_pack_plan_set_ptrs(kfac_pack_plan_t plan, const void *const *ptrs,
                            void *stream);
int64_t kfac_pack_plan_nelems(kfac_pack_plan_t plan);
int kfac_pack_plan_destroy(kfac_pack_plan_t plan);

/* buf[off_j + r(r+1)/2 + c] = M_j[r, c] for c <= r (triangular arrays), flat
 * copy otherwise; arrays whose rank differs from target_rank are skipped when
 * target_rank >= 0.  buf must be 16-byte aligned (8-byte for the float16
 * variant): the kernel stores aligned quads of buffer slots.  Triangle sides up
 * to 46340.  Replaces cupy_batched_pack_arrays and its launch
 * (pure_nccl_communicator.py:300-377, :110-127). */
int kfac_pack_f32(kfac_pack_plan_t plan, float *buf, int64_t buf_nelems,
                  int target_rank, void *stream);

/* M_j[r, c] = buf[off_j + tri(max(r,c), min(r,c))] / divisor for every r, c
 * (both triangles), flat arrays copied and divided.  Replaces
 * cupy_batched_unpack_arrays and its launch (pure_nccl_communicator.py:380-463,
 * :129-148). */
int kfac_unpack_f32(kfac_pack_plan_t plan, const float *buf, int64_t buf_nelems,
                    int target_rank, int divisor, void *stream);

/* The same with a float16 buffer (the arrays stay float32), the reference's
 * fp16 communication dtype: pack stores (half)value, round to nearest even
 * (pure_nccl_communicator.py:354-363); unpack divides in half precision,
 * buf[i] / (half)divisor, then widens (pure_nccl_communicator.py:438-449).
 * buf_nelems counts halves. */
int kfac_pack_f16(kfac_pack_plan_t plan, void *buf, int64_t buf_nelems,
                  int target_rank, void *stream);
int kfac_unpack_f16(kfac_pack_plan_t plan, const void *buf, int64_t buf_nelems,
                    int target_rank, int divisor, void *stream);

/* ------------------------------------------------------------------------
 * (1) Kronecker-factor construction:  C = beta*C + alpha * P^T P
 *     beta = 1, alpha = scale/acc_iters gives the running accumulation of
 *     optimizers/kfac.py:294-304; beta = 0 the plain covariance.
 *     All of them need kfac_cov_workspace_bytes(d, rows) bytes of workspace,
 *     d the side of C and rows the length of the reduction (samples, times
 *     output pixels for a convolution).  With less, a factor that has several
 *     routes takes one that fits (rows <= 0 asks for the bound of the routes
 *     whose need does not depend on it); with too little for any, the call
 *     fails with KFAC_ENOMEM.
 * --------------------------------------------------------------------- */
size_t kfac_cov_workspace_bytes(int d, int64_t rows);

/* P = [x, 1] (ones column last iff append_ones), x is (n, d_in) row-major.
 * With alpha = 1/n replaces FisherBlockLinear.compute_A
 * (optimizers/fisher_blocks/connections/linear.py:14-27); with x = gy,
 * append_ones = 0 and alpha = gy_scale^2/n replaces compute_G (:29-46); with
 * the (n, 2C) batch-norm gradient matrix it is the last step of compute_F. */
int kfac_cov_linear_f32(const float *x, int n, int d_in, int append_ones,
                        float alpha, float beta, float *C, void *ws,
                        size_t ws_bytes, void *stream);

/* P = im2col patches of the NCHW tensor x: rows (sample, y, x), columns
 * (c, kh, kw) then the ones column; zero padding, floor output size.  The
 * patch matrix is never materialised.  With alpha = 1/n replaces
 * FisherBlockConvolution2D.compute_A (connections/convolution_2d.py:19-41). */
int kfac_cov_conv_a_f32(const float *x, int n, int c, int h, int w, int kh,
                        int kw, int sy, int sx, int ph, int pw, int append_ones,
                        float alpha, float beta, float *C, void *ws,
                        size_t ws_bytes, void *stream);

/* Which kernels the calling thread's last kfac_cov_conv_a_f32 call used (the choice
 * depends on the geometry and, for the shifted correlations, on the size of the
 * workspace): for tests and benchmarks that must know a shape runs where they
 * think it does.  -1 before the first call.  No counterpart in the reference. */
#define KFAC_CONV_ROUTE_SLAB 0    /* 1x1 convolution: the NCHW tensor read in place        */
#define KFAC_CONV_ROUTE_SHIFT 1   /* 3x3 / 1 / 1: shifted correlations of the input       */
#define KFAC_CONV_ROUTE_ROWS 2    /* compile-time geometry, whole output rows per step     */
#define KFAC_CONV_ROUTE_HALO 3    /* halo regions staged in LDS                           */
#define KFAC_CONV_ROUTE_GATHER 4  /* implicit im2col, element gather                      */
int kfac_cov_conv_a_last_route(void);

/* P = gy viewed as (n*ho*wo, c) from the NCHW tensor gy, read in place.  With
 * alpha = gy_scale^2/(n*ho*wo) replaces compute_G (convolution_2d.py:43-72). */
int kfac_cov_conv_g_f32(const float *gy, int n, int c, int howo, float alpha,
                        float beta, float *C, void *ws, size_t ws_bytes,
                        void *stream);

/* The covariances of many (small) layers in a handful of launches.  A group is
 * created once for a list of items -- each what one kfac_cov_linear_f32 or
 * kfac_cov_conv_g_f32 / 1x1 kfac_cov_conv_a_f32 call would compute -- and run
 * with that call's pointers and alpha / beta per item:
 *   KFAC_COV_LINEAR  x (n, c) row-major: out = beta*out + alpha [x, 1]^T [x, 1]
 *                    (linear.py:14-46, and the last step of the batch-norm
 *                    factor, batch_normalization.py:121-131)
 *   KFAC_COV_SLAB    the (n, c, h, w) tensor read as rows = channels, reduction
 *                    over samples and pixels: the output-gradient factor of a
 *                    convolution (convolution_2d.py:43-72) and, with
 *                    append_ones, the input factor of a 1x1 convolution without
 *                    padding (convolution_2d.py:19-41); sy / sx > 1 take every
 *                    sy-th line and sx-th pixel (a strided 1x1 convolution).
 * `aligned` states that the item's input pointer will be 16-byte aligned (it is
 * then read with 16-byte loads where its strides allow).  The results are those
 * of the single calls up to the order of the floating-point sums.  Replaces the
 * per-layer loop over compute_A / compute_G / compute_F for layers too small to
 * fill the GPU one at a time; no single call of the reference corresponds.
 * The pointers and scales of a call travel to the GPU as a table; the group
 * keeps the last four distinct tables resident, so calls that alternate between
 * a few argument sets (beta = 0 on the first micro-batch, 1 afterwards) upload
 * nothing.  Under stream capture only a resident table can be used (call once
 * with the same arguments before capturing; KFAC_EINVAL otherwise), and a
 * captured graph keeps reading the table it was captured with: do not push it
 * out by running the same group with four other argument sets. */
#define KFAC_COV_LINEAR 0
#define KFAC_COV_SLAB 1
typedef struct kfac_cov_item {
  int32_t kind, n, c, h, w, sy, sx, append_ones, aligned;
} kfac_cov_item;
typedef struct kfac_cov_group *kfac_cov_group_t;
int kfac_cov_group_create(int count, const kfac_cov_item *items, kfac_cov_group_t *group_out);
size_t kfac_cov_group_workspace_bytes(kfac_cov_group_t group);
int kfac_cov_group_destroy(kfac_cov_group_t group);
/* A group runs its longest launch on the caller's stream and the others beside it on
 * a stream of its own, joined again before the call returns.  On a stream that is being
 * captured into a HIP graph it does so only after kfac_cov_group_set_capture_origin(group,
 * 1): the caller's statement that the stream is the one the capture began on (a stream
 * forked from a forked stream has crashed the runtime); otherwise every launch stays on
 * the given stream. */
int kfac_cov_group_set_capture_origin(kfac_cov_group_t group, int is_origin);
int kfac_cov_group_run_f32(kfac_cov_group_t group, const float *const *inputs,
                           float *const *outputs, const float *alpha, const float *beta,
                           void *ws, size_t ws_bytes, void *stream);

/* Per-sample batch-norm gradient matrix U (n, 2C) = [sum_hw gy'*h | sum_hw gy']
 * with h the batch-normalised x (biased variance, eps inside the root) and
 * gy' = gy*gy_scale; hw = 1 for 2-D inputs.  Only the gamma half / beta half
 * is written when has_beta / has_gamma is 0 (U is then (n, C)).  Replaces
 * normalizations/batch_normalization.py:86-119; follow with
 * kfac_cov_linear_f32(U, n, width, 0, 1/n, ...) for :121-131.
 * Workspace: kfac_bn_workspace_bytes(n, c). */
size_t kfac_bn_workspace_bytes(int n, int c);
int kfac_bn_grad_matrix_f32(const float *x, const float *gy, int n, int c,
                            int hw, float eps, float gy_scale, int has_gamma,
                            int has_beta, float *U, void *ws, size_t ws_bytes,
                            void *stream);

/* The same in two parts, so that the second part of every batch-norm layer of
 * a network is one launch.  kfac_bn_stats_f32: the pass over x and gy of one
 * layer, which leaves per (sample, channel) statistics in `stats`
 * (kfac_bn_workspace_bytes(n, c) bytes, kept by the caller until the finish).
 * kfac_bn_finish_batched_f32: U of `count` layers from their statistics; the
 * arithmetic of kfac_bn_grad_matrix_f32, bit-identical results.  Replaces the
 * loop over normalizations/batch_normalization.py:86-119 that the function
 * hook drives (optimizers/kfac.py:33-48).  The batch object keeps device
 * tables of the layers and rewrites them when the arguments change. */
int kfac_bn_stats_f32(const float *x, const float *gy, int n, int c, int hw,
                      float *stats, size_t stats_bytes, void *stream);
typedef struct kfac_bn_finish_batch *kfac_bn_finish_batch_t;
int kfac_bn_finish_batch_create(kfac_bn_finish_batch_t *batch_out);
int kfac_bn_finish_batch_destroy(kfac_bn_finish_batch_t batch);
int kfac_bn_finish_batched_f32(kfac_bn_finish_batch_t batch, int count,
                               const float *const *stats, float *const *U,
                               const int32_t *n, const int32_t *c,
                               const int32_t *hw, const float *eps,
                               const float *gy_scale, const int32_t *has_gamma,
                               const int32_t *has_beta, void *stream);

/* y = a*x + b*y over one pair of arrays of `nelems` floats; with b == 0, y is
 * overwritten without being read.
 * Moving average of optimizers/fisher_block.py:162-163 (a = decay on the new
 * covariance, b = 1-decay) and the unfused accumulation of kfac.py:286-304. */
int kfac_axpby_f32(const float *x, float *y, int64_t nelems, float a, float b,
                   void *stream);

/* The same for `count` pairs of arrays in one launch (one a and b for all):
 * the moving average of every factor of the network
 * (`for fblock in fblocks: fblock.update_cov_emas()`, kfac.py:306-308 over
 * fisher_block.py:155-163) or `accumulate_grads` over all parameters
 * (kfac.py:286-294).  Arrays need no alignment.  The batch object keeps the
 * device-side tables between calls and rewrites them only when the arguments
 * change (a rewrite synchronises the stream, and is refused while the stream
 * is being captured). */
typedef struct kfac_axpby_batch *kfac_axpby_batch_t;
int kfac_axpby_batch_create(kfac_axpby_batch_t *batch_out);
int kfac_axpby_batch_destroy(kfac_axpby_batch_t batch);
int kfac_axpby_batched_f32(kfac_axpby_batch_t batch, int count,
                           const float *const *xs, float *const *ys,
                           const int64_t *nelems, float a, float b, void *stream);

/* arrays[i][j] /= divisor (an IEEE division, like NumPy's in-place `/=`) for a list
 * of arrays in one launch: what Chainer's UpdateRule.update does to every
 * parameter's `grad` of a scaled loss before the rule runs (the reference's rule,
 * optimizers/kfac.py:63-85, does the same to `kfgrad`).  Takes a batch object of
 * kfac_axpby_batch_create. */
int kfac_div_batched_f32(kfac_axpby_batch_t batch, int count, float *const *arrays,
                         const int64_t *nelems, float divisor, void *stream);

/* ------------------------------------------------------------------------
 * (2) Damping and the damped inverse
 * --------------------------------------------------------------------- */

/* One plan per list of factor dimensions; holds the tile schedule on the
 * device.  The inverse of every matrix is potrf (blocked Cholesky) followed by
 * potri (triangular inverse, then L^-T L^-1), all matrices advancing together
 * one block column per launch. */
typedef struct kfac_inverse_plan *kfac_inverse_plan_t;

int kfac_inverse_plan_create(int count, const int32_t *dims,
                             kfac_inverse_plan_t *plan_out);
size_t kfac_inverse_plan_workspace_bytes(kfac_inverse_plan_t plan);
int kfac_inverse_plan_destroy(kfac_inverse_plan_t plan);

/* kfac_spd_inverse_batched_f32 runs part of its trailing updates on a stream
 * of the plan's own, forked from and joined back into `stream` with events.
 * While `stream` is being captured into a HIP graph that fork is only taken
 * when the caller has declared, with is_origin != 0, that `stream` is the
 * stream the capture began on; on any other capturing stream (one that itself
 * was forked into the capture) the call keeps all launches on `stream`.  The
 * results are the same either way.  No counterpart in the reference (which has
 * no stream structure). */
int kfac_inverse_plan_set_capture_origin(kfac_inverse_plan_t plan, int is_origin);

/* out_i = in_i^-1 for SPD in_i (dims given at plan creation); the full
 * symmetric inverse is written.  in_i is read only.  info_dev[i] (device,
 * int32) receives 0, or 1 + the index of the first non-positive pivot, which
 * the reference GPU path silently ignores (dev_info is never read,
 * optimizers/cholesky_inverse.py:42,94,100) and the NumPy path raises on.
 * Replaces inverse(a, use_cholesky=True) (cholesky_inverse.py:16-102) and the
 * per-factor loop of FisherBlock.update_invs (fisher_block.py:165-179). */
int kfac_spd_inverse_batched_f32(kfac_inverse_plan_t plan,
                                 const float *const *in_ptrs,
                                 float *const *out_ptrs, int32_t *info_dev,
                                 void *ws, size_t ws_bytes, void *stream);

/* Trace-norm pi and in-place damping of `count` (A, G) pairs:
 *   pi = float32(sqrt((tr A * dim G) / (tr G * dim A)))   (1 if !use_pi)
 *   diag(A) += pi*rW, diag(G) += rW/pi, the sums formed in float64 and
 *   rounded to float32 on store.
 * pi_out_dev (device, count floats, may be NULL) receives pi.
 * Replaces compute_pi_tracenorm (fisher_block.py:23-42),
 * FisherBlockConnection.get_diagvals (fisher_blocks/connection.py:66-77) and
 * the fill_diagonal of update_invs (fisher_block.py:175). */
typedef struct kfac_damp_plan *kfac_damp_plan_t;
int kfac_damp_plan_create(int count, const int32_t *dimsA, const int32_t *dimsG,
                          kfac_damp_plan_t *plan_out);
int kfac_damp_plan_destroy(kfac_damp_plan_t plan);
int kfac_pi_damp_batched_f32(kfac_damp_plan_t plan, float *const *A_ptrs,
                             float *const *G_ptrs, const double *rW, int use_pi,
                             float *pi_out_dev, void *stream);

/* Damped inverses of `count` batch-norm blocks from their low-rank form:
 * block i has the (n x widths[i]) per-sample gradient matrix U_i (row-major,
 * as written by kfac_bn_grad_matrix_f32) with factor F_i = U_i^T U_i / n, and
 *   out_i = (F_i + diag(d_gamma[i] for columns < splits[i], d_beta[i] after))^-1
 * as a dense symmetric (w x w) matrix, by the Woodbury identity (an n x n
 * Cholesky instead of a w^3 one).  n <= 32; the damping value of a half that
 * has columns must be positive.  info_dev[i] = 0, or 1 + the index of the
 * first non-positive pivot of the n x n matrix.  Mathematically the result of
 * update_invs (fisher_block.py:165-179, cholesky_inverse.py:16-102) on the
 * factor of normalizations/batch_normalization.py:121-131 damped per
 * batch_normalization.py:133-157; valid only while the block's moving average
 * is that single factor (cov_ema_decay == 1 or first step, no accumulation).
 * Workspace: kfac_bn_lowrank_workspace_bytes(plan). */
typedef struct kfac_bn_lowrank_plan *kfac_bn_lowrank_plan_t;
int kfac_bn_lowrank_plan_create(int count, int n, const int32_t *widths,
                                const int32_t *splits,
                                kfac_bn_lowrank_plan_t *plan_out);
size_t kfac_bn_lowrank_workspace_bytes(kfac_bn_lowrank_plan_t plan);
int kfac_bn_lowrank_plan_destroy(kfac_bn_lowrank_plan_t plan);
int kfac_bn_lowrank_inverse_batched_f32(kfac_bn_lowrank_plan_t plan,
                                        const float *const *U_ptrs,
                                        float *const *out_ptrs,
                                        const double *d_gamma, const double *d_beta,
                                        int32_t *info_dev, void *ws, size_t ws_bytes,
                                        void *stream);

/* diag(M)[i] += (i < split ? v0 : v1), float64 sum rounded to float32.
 * Batch-norm damping (normalizations/batch_normalization.py:133-157 with
 * fisher_block.py:175). */
int kfac_add_diag_f32(float *M, int d, int split, double v0, double v1,
                      void *stream);

/* M = diag(diag(M)): the off-diagonal entries of the d x d matrix are set to zero.
 * With the factor kernels before it, replaces `G = xp.diag(xp.diag(G))` of a link
 * with `diag` set (connections/convolution_2d.py:68-70) and the `diagonalize`
 * branches (convolution_2d.py:57-62, batch_normalization.py:121-124), whose
 * results are d x d matrices as well. */
int kfac_keep_diag_f32(float *M, int d, void *stream);

/* out[i] = 1 / (x[i] + (i < split ? v0 : v1)), evaluated in float64 and rounded to
 * float32: the inverse of a factor that is kept as its diagonal only (a 1-D
 * array), fisher_block.py:170-171, with the damping of kfac_add_diag_f32. */
int kfac_recip_add_f32(const float *x, int64_t split, double v0, double v1, float *out,
                       int64_t nelems, void *stream);

/* The same for `count` matrices in one launch (the damping of all batch-norm
 * blocks of a network: the loop of update_invs, fisher_block.py:165-179, over
 * normalizations/batch_normalization.py:133-157).  The batch object keeps the
 * argument table on the device; the last four distinct tables stay resident
 * (under stream capture only a resident table can be used). */
typedef struct kfac_diag_batch *kfac_diag_batch_t;
int kfac_diag_batch_create(kfac_diag_batch_t *batch_out);
int kfac_diag_batch_destroy(kfac_diag_batch_t batch);
int kfac_add_diag_batched_f32(kfac_diag_batch_t batch, int count, float *const *mats,
                              const int32_t *dims, const int32_t *splits, const double *v0,
                              const double *v1, void *stream);

/* ------------------------------------------------------------------------
 * (3) Preconditioning
 * --------------------------------------------------------------------- */

/* kf = (Ginv . [gradW | gradb]) . Ainv, the left product first;
 * kfW = kf[:, :dA-1] (or all of kf when gradb is NULL), kfb = kf[:, -1].
 * gradW is (dG, dA - has_bias) row-major (the weight gradient reshaped to
 * (c_out, -1)).  Workspace: kfac_precond_conn_workspace_bytes(dG, dA).
 * Replaces compute_kfgrads (connections/linear.py:48-61,
 * connections/convolution_2d.py:74-90) and the split of
 * FisherBlockConnection.update_kfgrads (fisher_blocks/connection.py:51-61). */
size_t kfac_precond_conn_workspace_bytes(int dG, int dA);
int kfac_precond_conn_f32(const float *Ginv, int dG, const float *Ainv, int dA,
                          const float *gradW, const float *gradb, float *kfW,
                          float *kfb, void *ws, size_t ws_bytes, void *stream);

/* kfac_precond_conn_f32 for all connection layers of a network in a few
 * launches: a group is created once for the layers' (dG, dA, has_bias) and run
 * with one pointer per layer and operand (gradb[i] / kfb[i] NULL where the layer
 * has no bias; all pointers 16-byte aligned).  The two products of every layer
 * are cut into tasks of about equal length and run from task tables: first
 * Ginv . [gradW | gradb] of all layers, then . Ainv of all layers.  Results as
 * kfac_precond_conn_f32 up to the order of the floating-point sums.  Replaces
 * the loop over fblock.update_kfgrads() (optimizers/kfac.py:306-310) for the
 * connection blocks. */
typedef struct kfac_precond_group *kfac_precond_group_t;
int kfac_precond_group_create(int count, const int32_t *dG, const int32_t *dA,
                              const int32_t *has_bias, kfac_precond_group_t *group_out);
size_t kfac_precond_group_workspace_bytes(kfac_precond_group_t group);
int kfac_precond_group_destroy(kfac_precond_group_t group);
/* Like a covariance group, a preconditioning group runs the longest launch of each
 * phase on the caller's stream and the others on a stream of its own; under stream
 * capture only after the caller has declared the stream the capture's origin. */
int kfac_precond_group_set_capture_origin(kfac_precond_group_t group, int is_origin);
int kfac_precond_group_run_f32(kfac_precond_group_t group, const float *const *Ginv,
                               const float *const *Ainv, const float *const *gradW,
                               const float *const *gradb, float *const *kfW,
                               float *const *kfb, void *ws, size_t ws_bytes, void *stream);

/* kf = Finv . [g_gamma ; g_beta] split at n_gamma; if any element of kf is
 * NaN every output is the raw gradient instead and *nan_flag_dev (device
 * int32, may be NULL) is set to 1, else 0.  Either half may be absent
 * (pointer NULL, size 0).  Workspace: d floats + 1 int.
 * Replaces batch_normalization.py:159-191 and _check_nan (:21-33). */
size_t kfac_precond_bn_workspace_bytes(int d);
int kfac_precond_bn_f32(const float *Finv, int d, const float *g_gamma,
                        int n_gamma, const float *g_beta, int n_beta,
                        float *kf_gamma, float *kf_beta, int32_t *nan_flag_dev,
                        void *ws, size_t ws_bytes, void *stream);

/* kfac_precond_bn_f32 for a list of batch-norm blocks in two launches (the products
 * of all blocks, then the NaN selection of all blocks) instead of two per block;
 * the arithmetic is the single-block kernels' own, so the results are identical.
 * Block i: Finv[i] (dims[i] x dims[i]), gradients g_gamma[i] (n_gamma[i] entries)
 * and g_beta[i] (the rest), outputs kf_gamma[i] / kf_beta[i], flag nan_flags[i]
 * (device int32; the table or an entry may be NULL).  The batch object keeps the
 * device-side tables between calls and uploads them again, with copies ordered on
 * `stream`, only when the arguments change.  Workspace: the sum of the dims
 * rounded up to multiples of 4, in floats.
 * Replaces the per-block loop over batch_normalization.py:159-191 of
 * optimizers/kfac.py:306-310. */
typedef struct kfac_precond_bn_batch *kfac_precond_bn_batch_t;
int kfac_precond_bn_batch_create(kfac_precond_bn_batch_t *batch_out);
int kfac_precond_bn_batch_destroy(kfac_precond_bn_batch_t batch);
size_t kfac_precond_bn_batched_workspace_bytes(int count, const int32_t *dims);
int kfac_precond_bn_batched_f32(kfac_precond_bn_batch_t batch, int count,
                                const float *const *Finv, const int32_t *dims,
                                const float *const *g_gamma, const int32_t *n_gamma,
                                const float *const *g_beta, float *const *kf_gamma,
                                float *const *kf_beta, int32_t *const *nan_flags,
                                void *ws, size_t ws_bytes, void *stream);

/* kfac_precond_bn_f32 without a workspace argument and without any allocation:
 * the staging vector lives in a device array of KFAC_PRECOND_BN_STATIC_MAX_D
 * floats (32 KiB) that is part of the library image on every GPU the library
 * runs on, for the life of the process.  No counterpart in the reference; it is
 * for callers that cannot allocate device memory -- code under HIP-graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  The call makes
 * no hipMalloc/hipFree and calls no allocating library routine; inputs and
 * outputs are the caller's, as for kfac_precond_bn_f32, and the results are
 * identical to it.  d > KFAC_PRECOND_BN_STATIC_MAX_D is rejected with
 * KFAC_EINVAL.  The first call on a device looks up the array's address on that
 * device (hipGetSymbolAddress, once): make one call outside of any stream
 * capture first.  All calls on one GPU share the one array: calls that may
 * overlap on the same GPU (different streams, different threads) race on it and
 * must be serialised by the caller. */
#define KFAC_PRECOND_BN_STATIC_MAX_D 8192
int kfac_precond_bn_static_f32(const float *Finv, int d, const float *g_gamma,
                               int n_gamma, const float *g_beta, int n_beta,
                               float *kf_gamma, float *kf_beta,
                               int32_t *nan_flag_dev, void *stream);

/* v = momentum*v - lr*grad; param += v.  Replaces the 'kfac' elementwise
 * kernel of KFACUpdateRule.update_core_gpu (optimizers/kfac.py:101-116). */
int kfac_momentum_update_f32(float *param, float *v, const float *grad,
                             int64_t nelems, float lr, float momentum,
                             void *stream);

/* The same rule for many parameters in one launch, with the loss-scale and
 * float16 handling of KFACUpdateRule.update (optimizers/kfac.py:63-85) folded
 * in.  For every element of parameter i:
 *   g = grads[i][e] (float32, or float16 with KFAC_MOMENTUM_GRAD_F16);
 *   if loss_scale != 1:  g = g / loss_scale (an IEEE division), and with
 *     KFAC_MOMENTUM_WRITE_BACK_GRAD and a float32 gradient the quotient is
 *     stored back (the reference divides `kfgrad` in place, kfac.py:76-78);
 *   v = momentum*v - lr*g;  params[i][e] += v  (float32: the master copy of a
 *     float16 parameter, kfac.py:64-68);
 *   if params_f16 and params_f16[i]:  params_f16[i][e] = float16(params[i][e])
 *     (what Chainer's use_fp32_update copies back into the parameter).
 * lr and momentum are common to the call: parameters whose rules carry other
 * hyperparameters go into a call of their own.  `flags` and `params_f16` may
 * be null.  Arrays need no alignment (16-byte aligned ones are moved 16 bytes
 * per lane).  The batch object keeps the device-side tables between calls and
 * rewrites them only when the arguments change (a rewrite synchronises the
 * stream, and is refused while the stream is being captured). */
typedef struct kfac_momentum_batch *kfac_momentum_batch_t;
#define KFAC_MOMENTUM_GRAD_F16 1
#define KFAC_MOMENTUM_WRITE_BACK_GRAD 2
int kfac_momentum_batch_create(kfac_momentum_batch_t *batch_out);
int kfac_momentum_batch_destroy(kfac_momentum_batch_t batch);
int kfac_momentum_update_batched_f32(kfac_momentum_batch_t batch, int count,
                                     float *const *params, float *const *vs,
                                     void *const *grads, const int64_t *nelems,
                                     const int32_t *flags, void *const *params_f16,
                                     float lr, float momentum, float loss_scale,
                                     void *stream);

/* ------------------------------------------------------------------------
 * Per-kernel timing for benchmarks (no counterpart in the reference, which
 * has no instrumentation).  While enabled, every launch of the kernel
 * families below is bracketed by a pair of HIP events on its own stream.
 * kfac_timing_read waits for the recorded events, adds their elapsed times to
 * the family totals and returns the totals since the last enable.
 * --------------------------------------------------------------------- */
#define KFAC_TIMED_SYRK 0      /* covariance main kernel (all loaders)        */
#define KFAC_TIMED_INV_UPDATE 1 /* inverse: trailing tile update kernel       */
#define KFAC_TIMED_INV_LAUUM 2  /* inverse: final U U^T kernel                */
#define KFAC_TIMED_GEMM 3       /* preconditioning GEMM kernel                */
#define KFAC_TIMED_PACK 4       /* pack kernel                                */
#define KFAC_TIMED_UNPACK 5     /* unpack kernel                              */
#define KFAC_TIMED_COPY 6       /* kfac_stream_copy_f32                        */
#define KFAC_TIMED_COV_AUX 7    /* covariance: kernels around the main one (border sums, split-K sums,
                                   assembly of a factor from shifted correlations)                     */
#define KFAC_TIMED_BN 8         /* batch-norm statistics and per-sample gradient matrix               */
#define KFAC_TIMED_INV_CALL 9   /* one whole kfac_spd_inverse_batched_f32 call: first launch to last  */
#define KFAC_TIMED_GEMM_AUX 10  /* preconditioning: split-K sums and the batch-norm GEMV              */
#define KFAC_TIMED_FAMILIES 11

/* dst[i] = src[i] for nelems floats (16-byte aligned pointers): a plain
 * streaming copy that moves 8 bytes per element, the yardstick that bench.py
 * puts beside the pack / unpack bandwidth (what a copy kernel reaches on the
 * same GPU in the same run).  No counterpart in the reference. */
int kfac_stream_copy_f32(float *dst, const float *src, int64_t nelems, void *stream);

/* dst0[i] = dst1[i] = src[i]: the same streaming kernel with the traffic mix of the
 * unpack kernel (every packed element is read once and, but for the diagonal,
 * written twice: 12 bytes per element), as a second yardstick.  nelems a multiple
 * of 4, 16-byte aligned pointers.  No counterpart in the reference. */
int kfac_stream_fanout_f32(float *dst0, float *dst1, const float *src, int64_t nelems,
                           void *stream);

int kfac_timing_enable(int on);
int kfac_timing_read(int family, int64_t *launches, double *total_ms);

#ifdef __cplusplus
}
#endif
#endif /* KFAC_HIP_H_ */
