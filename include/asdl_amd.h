/*
 * asdl_amd.h -- C ABI of the MI355X (gfx950) kernels behind the K-FAC / Shampoo
 * curvature path of kazukiosawa/asdl.
 *
 * The reference has no FFI: its hot path is a chain of ATen calls made from Python.
 * Each entry point below replaces one such chain; the comment above it cites the
 * reference lines (paths relative to the reference checkout).
 *
 * Conventions
 *   - Every pointer except `const char*` results is a DEVICE pointer unless stated.
 *   - Matrices are row-major with an explicit leading dimension in elements.
 *   - `stream` is a hipStream_t passed as void*; NULL is the default stream.  All work
 *     is enqueued on that stream; no entry point synchronises the device.
 *   - The caller owns every buffer, including workspaces.  Workspace sizes come from
 *     the matching ak_*_ws_bytes() query.  Nothing here allocates or frees device memory.
 *   - Return value: 0 ok; <0 bad argument (see ak_error_string).  Numerical failures
 *     (non positive-definite input) are reported through a device `info` word, like
 *     LAPACK's info, because they are only known once the stream has run.
 *   - Thread safety: entry points may be called from any host thread (autograd hooks run on the
 *     engine's device thread).  The only state the library keeps is caches behind mutexes (memoised
 *     launch plans keyed by problem shape) and the per-device address of the static scratch array of
 *     ak_kron_precond_static; no setter changes its behaviour (tuning setters exist only in builds
 *     with -DAK_TUNING_HOOKS, which is not how the shipped library is built).
 */
#ifndef ASDL_AMD_H
#define ASDL_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AK_F32 0
#define AK_BF16 1
#define AK_F32_AS_BF16 2     /* fp32 in memory, every element rounded to the nearest bf16 (ties to even) as it is read:
                                what torch.matmul does to an fp32 operand inside a bf16 autocast region, where the
                                reference's hooks run.  ak_conv_syrk / ak_conv_syrk_nhwc only, and only for layers of
                                the window kernel (C*kh*kw <= 160, kh*kw > 1); AK_ERR_UNSUPPORTED elsewhere */

#define AK_OK 0
#define AK_ERR_ARG -1        /* null pointer, negative size, unknown dtype */
#define AK_ERR_WORKSPACE -2  /* workspace missing or too small */
#define AK_ERR_UNSUPPORTED -3
#define AK_ERR_LAUNCH -4     /* hipGetLastError() reported a launch failure */
#define AK_ERR_TOO_LARGE -5  /* sizes beyond the fixed maximum of an entry point that brings its own scratch memory */

typedef void* ak_stream_t;

int ak_version(void);
const char* ak_error_string(int code);

/* ---- Kronecker-factor statistics -------------------------------------------------- */

/* C <- beta*C + alpha * X^T X, X = [M, d] row-major (leading dimension ldx), C = [d, d] fp32,
 * full symmetric on exit (upper triangle computed, mirrored).  beta == 0 never reads C; beta != 0 needs C below
 * 4 GiB (d < 32768 for ldc == d), else AK_ERR_UNSUPPORTED: this holds for all three statistics entry points.
 * Replaces Linear.cov_kron_A / cov_kron_B  (asdl/operations/linear.py:75-77, 87-89), the
 * `.mul_(cov_scale)` and `results[key] += value` passes (asdl/operations/operation.py:133-137,
 * 199-201, 264-266) and the EMA pre-scale Kron.mul_ (asdl/symmatrix.py:448-453), and the 2-D
 * statistic G^T G of Shampoo (asdl/precondition/shampoo.py:331-339). */
size_t ak_syrk_tn_ws_bytes(int64_t M, int64_t d);
int ak_syrk_tn(const void* X, int dtype, int64_t M, int64_t d, int64_t ldx,
               float alpha, float beta, float* C, int64_t ldc,
               void* ws, size_t ws_bytes, ak_stream_t stream);

/* A <- beta*A + alpha * sum_{n,oy,ox} p p^T with p the (c,ky,kx)-ordered patch of x at output
 * position (oy,ox): the unfold is fused, the [n, c*kh*kw, h_out*w_out] tensor is never written.
 * x = [N, C, H, W] contiguous NCHW, zero padding (ph,pw), stride (sh,sw), dilation 1, groups 1.
 * A = [d, d] fp32 with d = C*kh*kw.  The caller folds 1/out_size into alpha.
 * Replaces im2col_2d (asdl/utils.py:51-71) + Conv2d.cov_kron_A (asdl/operations/conv.py:80-88).
 * With kh=kw=1, H=1, W=h_out*w_out it is sum_n G_n G_n^T for out_grads [N, C, hw], i.e.
 * Conv2d.cov_kron_B (asdl/operations/conv.py:99-103), and with N=1 it is X X^T for a row-major
 * [d, M] matrix (Shampoo's G G^T, asdl/precondition/shampoo.py:331-339). */
size_t ak_conv_syrk_ws_bytes(int64_t N, int64_t C, int64_t H, int64_t W,
                             int kh, int kw, int sh, int sw, int ph, int pw);
int ak_conv_syrk(const void* x, int dtype, int64_t N, int64_t C, int64_t H, int64_t W,
                 int kh, int kw, int sh, int sw, int ph, int pw,
                 float alpha, float beta, float* A, int64_t lda,
                 void* ws, size_t ws_bytes, ak_stream_t stream);

/* Same statistic as ak_conv_syrk for a channels-last input: x = [N, H, W, C] contiguous (the memory of a
 * torch.channels_last NCHW tensor), bf16, C a multiple of 8.  Rows of the unfolded input are gathered
 * straight from x; A is written in the same (c,ky,kx) order as ak_conv_syrk, so both entry points
 * are interchangeable replacements of im2col_2d (asdl/utils.py:51-71) + Conv2d.cov_kron_A
 * (asdl/operations/conv.py:80-88).  AK_ERR_UNSUPPORTED for other dtypes, channel counts or tensors
 * of 4 GiB and more: callers then use ak_conv_syrk on an NCHW copy. */
size_t ak_conv_syrk_nhwc_ws_bytes(int64_t N, int64_t C, int64_t H, int64_t W,
                                  int kh, int kw, int sh, int sw, int ph, int pw);
int ak_conv_syrk_nhwc(const void* x, int dtype, int64_t N, int64_t C, int64_t H, int64_t W,
                      int kh, int kw, int sh, int sw, int ph, int pw,
                      float alpha, float beta, float* A, int64_t lda,
                      void* ws, size_t ws_bytes, ak_stream_t stream);

/* The statistics of many layers in one launch sequence: what ak_syrk_tn (bf16 operand, 16-byte aligned rows) and
 * ak_conv_syrk_nhwc compute one factor at a time, i.e. Linear / Conv2d cov_kron_A and cov_kron_B
 * (asdl/operations/linear.py:75-89, asdl/operations/conv.py:80-103) of a whole forward or backward pass, whose
 * hooks the reference runs one by one (asdl/core.py:41-62).  Taken one at a time these factors are launches of a
 * few tiles, split along the rows to fill the device; together they fill it with long work items and few splits.
 * specs: HOST array of n rows of 16 int64:
 *   [0] kind: 0 = X^T X of a bf16 [M, d] matrix, 1 = unfolded channels-last bf16 [N, C, H, W] input
 *   [1] operand address (device)  [2] result address (device, fp32 [d, d])  [3] ldc
 *   [4] alpha (float bits, low word) and beta (float bits, high word): result <- beta*result + alpha*statistic
 *   kind 0: [5] M  [6] d  [7] ldx      kind 1: [5] N  [6] C  [7] H  [8] W  [9] kh  [10] kw  [11] sh  [12] sw  [13] ph  [14] pw
 * ak_syrk_group_eligible: 1 when the row can be part of a group (else use the single-factor entry points: fp32
 * operands, unaligned rows, few input channels, factors of 3456 columns and more).
 * ak_syrk_group_sizes: bytes of the descriptor tables and of the workspace (partial tiles) of a group.
 * ak_syrk_group_launch: host_stage is HOST memory of table_bytes (pinned, so that the copy is asynchronous) that
 * the caller leaves alone until the stream has passed the copy; dev_tables and ws are device memory.  Two rows with
 * the same result address are refused (AK_ERR_ARG): they would race.  Fixed summation order: results are
 * reproducible bit for bit for a given list of shapes. */
int ak_syrk_group_eligible(const int64_t* spec);
int ak_syrk_group_sizes(const int64_t* specs, int n, size_t* table_bytes, size_t* ws_bytes);
int ak_syrk_group_launch(const int64_t* specs, int n, void* host_stage, void* dev_tables, size_t table_bytes,
                         void* ws, size_t ws_bytes, ak_stream_t stream);

/* ---- damping ---------------------------------------------------------------------- */

/* For each pair b < batch: tr(A_b), tr(B_b), the pi split
 *   pi = sqrt((trA/dA)/(trB/dB)); lamA = max(sqrt(damping)*pi, eps), lamB = max(sqrt(damping)/pi, eps)
 *   (lamA = lamB = damping when pi is 0 or inf), and the all-zero test of each factor.
 * A_list / B_list: device arrays of device pointers (dense, ld = dim).  dims: device int64 [batch,2].
 * lam_out: device float [batch,2]; nonzero_out: device int [batch,2] (1 when the factor has a
 * non-zero entry).  One launch, no host synchronisation.
 * Replaces the head of Kron.update_inv (asdl/symmatrix.py:499-510, 516, 527) and
 * Operation.cov_kron_damping (asdl/operations/operation.py:457-466). */
int ak_kron_damping(const float* const* A_list, const float* const* B_list, const int64_t* dims,
                    int batch, float damping, float eps, float* lam_out, int* nonzero_out,
                    ak_stream_t stream);

/* ---- low-rank ("swift") Kronecker factors --------------------------------------------- */

/* X[n][(c,ky,kx)] <- beta*X + alpha * sum over output positions of the patch element of sample n, read straight
 * from the activation x[n][c][iy][ix] with element strides (sn, sc, sh_el, sw_el): the n x d matrix SKFAC keeps
 * in place of a d x d factor when n < d.  With kh = kw = 1 it is the sum over positions (of an output gradient),
 * with H = W = 1 a scaled fp32 copy (Linear).  X = [N, ldo] fp32.
 * Replaces Conv2d.cov_swift_kron_A / _B (asdl/operations/conv.py:90-111: `in_data.sum(dim=-1)` of the unfolded
 * input, `out_grads.sum(dim=-1)`) and Linear.cov_swift_kron_A / _B (asdl/operations/linear.py:79-97). */
int ak_conv_patch_sum(const void* x, int dtype, int64_t sn, int64_t sc, int64_t sh_el, int64_t sw_el,
                      int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw, int ph, int pw,
                      float alpha, float beta, float* out, int64_t ldo, ak_stream_t stream);

/* out_list[m] (device array of `count` pointers to contiguous fp32 [dims[m], dims[m]] matrices) <- the identity
 * where nonzero[flag_index[m]] == 0, i.e. where ak_kron_damping found the factor all zero; the other matrices are not
 * touched.  dims, flag_index: device int64 [count]; nonzero: the device flags ak_kron_damping wrote.
 * The reference skips the inverse of an all-zero factor on the host (`if not torch.all(self.A == 0)`,
 * asdl/symmatrix.py:517, :527); a caller that does not want to read the flags before it preconditions lets such a
 * factor precondition with the identity instead. */
int ak_identity_where_zero(float* const* out_list, const int64_t* dims, const int* nonzero,
                           const int64_t* flag_index, int count, ak_stream_t stream);

/* ak_kron_damping for pairs whose factors may be n x d row matrices: dims = device int64 [batch,4]
 * (rows_A, d_A, rows_B, d_B; rows = 0: square d x d factor, eigenvalue mean trace/d; rows > 0: sum(x^2)/d),
 * eig_scale = device float [batch,2] multiplied into the eigenvalue means (may be null).
 * Replaces Operation.cov_kron_damping (asdl/operations/operation.py:457-466) and the head of Kron.update_inv
 * (asdl/symmatrix.py:499-510) for non-square factors. */
int ak_kron_damping_swift(const float* const* A_list, const float* const* B_list, const int64_t* dims,
                          const float* eig_scale, int batch, float damping, float eps, float* lam_out,
                          int* nonzero_out, ak_stream_t stream);

/* Z <- (I - Z) / lam[0], Z = [d, d] fp32 with row stride ld, lam in device memory: the last step of
 * smw_inv (asdl/utils.py:107-115), whose products run in ak_conv_syrk (x x^T), ak_chol_inv_batched and
 * ak_gemm_f32. */
int ak_smw_finish(float* Z, int64_t d, int64_t ld, const float* lam, ak_stream_t stream);

/* out <- (x^T x / n + lam[0] I)^-1 for x = [n, d] fp32 dense (n < d), lam in device memory: the whole of smw_inv
 * (asdl/utils.py:107-115) in one call -- Gram matrix x x^T + n lam I, its Cholesky inverse (info[0] as in
 * ak_chol_inv_batched), G^-1 x, x^T G^-1 x and the final (I - .) / lam, all enqueued on `stream`.
 * ws: 256-byte aligned, ak_smw_inv_ws_bytes(n, d) bytes. */
size_t ak_smw_inv_ws_bytes(int64_t n, int64_t d);
int ak_smw_inv(const float* x, int64_t n, int64_t d, const float* lam, float* out, int64_t ldo, int* info,
               void* ws, size_t ws_bytes, ak_stream_t stream);

/* ---- damped inverse --------------------------------------------------------------- */

/* out_b <- (A_b + lam_b I)^-1 for b < batch; all matrices d x d fp32 dense (ld = d); A_b is not
 * modified.  Blocked Cholesky (LDS-resident diagonal blocks, fp32 MFMA panel/trailing updates),
 * triangular inverse, and L^-T L^-1, all on `stream`.  lam: device float array with element
 * stride lam_stride.  info: device int [batch]; 0 ok, k > 0 means the leading minor of order k is
 * not positive definite (LAPACK potrf convention); out_b is then undefined.  If skip_flags is
 * non-NULL (device int, stride skip_stride) matrices whose flag is 0 are left untouched
 * (the reference skips all-zero factors).
 * Replaces cholesky_inv (asdl/utils.py:91-96) as called from asdl/symmatrix.py:518, 529 and
 * asdl/operations/operation.py:273-275. */
size_t ak_chol_inv_ws_bytes(int64_t d, int batch);
int ak_chol_inv_batched(const float* const* A_list, float* const* out_list, int64_t d, int batch,
                        const float* lam, int lam_stride, const int* skip_flags, int skip_stride,
                        int* info, void* ws, size_t ws_bytes, ak_stream_t stream);

/* ak_chol_inv_batched for `count` matrices of different sizes dims[m] in one call: the per-matrix sequences of
 * steps (LDS-resident diagonal block | panel and trailing products) are merged into one sequence of grouped
 * launches, so that the chains of the small matrices run in the shadow of the largest one's and nothing waits on
 * the host (ResNet-50: 156 factors of 13 sizes, about 150 launches).  The launch plan depends on the sizes only:
 *   ak_chol_group_plan_bytes / ak_chol_group_ws_bytes  bytes of the plan / of the device workspace (0: bad sizes);
 *   ak_chol_group_plan        fills plan_host (HOST memory); the caller keeps it and a byte copy in device memory;
 *   ak_chol_group_plan_launches  kernel launches one call enqueues;
 *   ak_chol_inv_grouped       plan_host and plan_dev are those two copies; A_list / out_list: device arrays of
 *                             `count` device pointers (dense, ld = dims[m]); lam, skip_flags, info as in
 *                             ak_chol_inv_batched, indexed by m; ws 256-byte aligned.
 * Only the lower triangle of A_m is read; out_m is written in full (both triangles).
 * Same reference lines as ak_chol_inv_batched; the loop it replaces is the per-module Kron.update_inv of
 * NaturalGradientMaker.update_preconditioner (asdl/precondition/natural_gradient.py:419-443). */
size_t ak_chol_group_plan_bytes(const int64_t* dims, int count);
size_t ak_chol_group_ws_bytes(const int64_t* dims, int count);
int ak_chol_group_plan(const int64_t* dims, int count, void* plan_host, size_t plan_bytes);
int ak_chol_group_plan_launches(const void* plan_host);
int ak_chol_inv_grouped(const void* plan_host, const void* plan_dev, const float* const* A_list,
                        float* const* out_list, const float* lam, int lam_stride, const int* skip_flags,
                        int skip_stride, int* info, void* ws, size_t ws_bytes, ak_stream_t stream);

/* ---- unit-wise blocks (BatchNorm / LayerNorm) ------------------------------------- */

/* blocks[f] <- beta*blocks[f] + alpha * sum_n [[gw^2, gw*gb], [gw*gb, gb^2]] for f < F, blocks = [F, 2, 2] fp32,
 * with gw[n,f] = sum_s (y[n,f,s] - bias[f]) / weight[f] * g[n,f,s] and gb[n,f] = sum_s g[n,f,s].
 * y is the module's output, g the gradient with respect to it; both fp32 or bf16, addressed through element
 * strides for (sample n, feature f, position s), so NCHW, channels-last and [rows, features] (S = 1) layouts
 * are read in place.  Replaces _BatchNormNd.preprocess_in_data + cov_unit_wise
 * (asdl/operations/batchnorm.py:11-21, 28-55, 95-108), LayerNorm.preprocess_in_data + cov_unit_wise
 * (asdl/operations/layernorm.py:20-31, 75-84) and the .mul_(cov_scale) / accumulate of
 * asdl/operations/operation.py:308-316. */
size_t ak_unit_wise_ws_bytes(int64_t N, int64_t F, int64_t S);
int ak_unit_wise_stats(const void* y, int y_dtype, int64_t ysn, int64_t ysf, int64_t yss,
                       const void* g, int g_dtype, int64_t gsn, int64_t gsf, int64_t gss,
                       const float* weight, const float* bias, int64_t N, int64_t F, int64_t S,
                       float alpha, float beta, float* blocks,
                       void* ws, size_t ws_bytes, ak_stream_t stream);

/* inv[f] <- (blocks[f] + damping I)^-1 for the F 2x2 blocks.  flags: device int[2]; flags[0] = 1 when blocks has a
 * non-zero entry (the reference skips the inverse of an all-zero tensor), flags[1] = 1-based index of the first
 * singular block or 0x7fffffff.  Replaces UnitWise.update_inv (asdl/symmatrix.py:687-699) and the inverse of
 * asdl/operations/operation.py:317-321. */
int ak_unit_wise_inv(const float* blocks, int64_t F, float damping, float* inv, int* flags, ak_stream_t stream);

/* ak_unit_wise_inv for many modules in one launch.  `table` is DEVICE memory, `count` rows of 6 int64: blocks,
 * inv, flags (addresses; the caller presets each flags pair to {0, 0x7fffffff}), F, first_block (running sum of
 * ceil(F/256)), damping (float bit pattern in the low 32 bits).  Same reference lines as ak_unit_wise_inv. */
int ak_unit_wise_inv_grouped(const int64_t* table, int count, int64_t total_blocks, ak_stream_t stream);

/* [vec_weight[f], vec_bias[f]] <- mat[f] @ (scale * [vec_weight[f], vec_bias[f]]) in place, mat = [F, 2, 2].
 * Replaces UnitWise.mvp for BatchNorm / LayerNorm (asdl/symmatrix.py:701-709, 716-719) and the grad_scale
 * pre-multiply of asdl/precondition/natural_gradient.py:535-538. */
int ak_unit_wise_mvp(const float* mat, int64_t F, float* vec_weight, float* vec_bias, float scale,
                     ak_stream_t stream);

/* ak_unit_wise_mvp for many modules in one launch.  `table` is DEVICE memory, `count` rows of 5 int64: mat,
 * vec_weight, vec_bias (addresses), F, first_block (running sum of ceil(F/256)); total_blocks that sum over all
 * rows.  The unit-wise modules of the loop at asdl/precondition/natural_gradient.py:481-486. */
int ak_unit_wise_mvp_grouped(const int64_t* table, int count, int64_t total_blocks, float scale, ak_stream_t stream);

/* ---- saved factors ----------------------------------------------------------------- */

/* tril[i*(i+1)/2 + j] = mat[i][j] for j <= i (row direction), the 1-D form in which factors are saved as
 * float32 .npy files; and the inverse, which fills both triangles.  d <= 65535.
 * Replaces matrix_to_tril / tril_to_matrix (asdl/symmatrix.py:25-54) as used by SymMatrix.save / load and
 * Kron.save / load (asdl/symmatrix.py:226-269, 471-492). */
int ak_tril_pack(const float* mat, int64_t d, int64_t ld, float* tril, ak_stream_t stream);
int ak_tril_unpack(const float* tril, int64_t d, float* mat, int64_t ld, ak_stream_t stream);

/* ---- dense fp32 products ---------------------------------------------------------- */

/* C <- alpha * op(A) op(B) + beta * C, fp32 MFMA, row-major; op = identity (0) or transpose (1);
 * C = [M, N], op(A) = [M, K], op(B) = [K, N].  batch > 1 strides all three by the given element
 * strides.  Replaces the mm calls of Kron.mvp (asdl/symmatrix.py:536-548), the tensordot chain of
 * Preconditioner.precondition (asdl/precondition/shampoo.py:351-367) and the matmuls of
 * ComputePower / MatPower (asdl/precondition/shampoo.py:518-527, 561-586). */
int ak_gemm_f32(int transA, int transB, int64_t M, int64_t N, int64_t K, float alpha,
                const float* A, int64_t lda, const float* B, int64_t ldb, float beta,
                float* C, int64_t ldc, int batch, int64_t strideA, int64_t strideB, int64_t strideC,
                ak_stream_t stream);

/* The same product on the bf16 matrix cores: each fp32 operand element is split exactly into `pieces`
 * bf16 values (3: all 24 mantissa bits, six partial products, error of the order of an fp32 multiply;
 * 2: 16 bits, three partial products) and accumulated in fp32.  pieces = 0 is ak_gemm_f32.  Operands that
 * the split kernel cannot take (leading dimensions or inner extents not multiples of 4, small shapes)
 * are multiplied by the fp32 MFMA kernel.  Same reference call sites as ak_gemm_f32. */
int ak_gemm_f32_split(int pieces, int transA, int transB, int64_t M, int64_t N, int64_t K, float alpha,
                const float* A, int64_t lda, const float* B, int64_t ldb, float beta,
                float* C, int64_t ldc, int batch, int64_t strideA, int64_t strideB, int64_t strideC,
                ak_stream_t stream);

/* Many products of different sizes in one launch: C_i <- alpha_i * op(A_i) op(B_i) + beta_i * C_i on the bf16
 * matrix cores (pieces = 2 or 3 as in ak_gemm_f32_split) or with true fp32 products (pieces = 0, the fp32 MFMA, one
 * accumulation per k; needs no alignment), or on two fp16 pieces per element (pieces = 22: 22 significant bits, three
 * partial products; each operand is multiplied by the power of two that brings its largest magnitude, read from the
 * float word absmax_A / absmax_B names, into (2^13, 2^14]; pieces = 23: the same, summed in chunks of 256 k: the
 * products of the leading pieces in an accumulator of their own that joins a running total, which keeps the rounding
 * of a long sum near that of a single one).  `table` is DEVICE memory, `count` rows of 16 int64:
 *   A, B, C (addresses), lda, ldb, ldc, M, N, K, transA | transB << 1 | symmetric << 2, alpha and beta (float
 *   bit patterns in the low and the high 32 bits), first_tile, absmax_A, absmax_B, absmax_C, 0
 * (absmax_A, absmax_B: addresses of float words, required for pieces = 22 and 23, ignored otherwise; absmax_C: 0 or the
 * address of a float word into which the split kernels fold max |C_i| by an integer atomic maximum on the bit pattern:
 * zero it first)
 * (symmetric: M == N and op(A) op(B) is symmetric, e.g. G G^T: only the tiles on and below the diagonal are
 * computed and mirrored, the result is exactly symmetric)
 * with first_tile the running sum of ceil(M/128) * ceil(N/128) over the rows before, and total_tiles that sum
 * over all rows.  Every operand has to satisfy what the split kernel needs (16-byte aligned addresses, leading
 * dimensions and the contiguous extents of both operands multiples of 4); the table cannot be checked from the
 * host.  Rows sorted by descending K balance best.  Replaces the per-module loop around Kron.mvp of
 * NaturalGradientMaker.precondition (asdl/precondition/natural_gradient.py:481-486, asdl/symmatrix.py:536-548):
 * one call computes Binv_i G_i for every module, a second one (.) Ainv_i; and the tensordot(G, G) statistics and
 * the per-axis preconditioning of all matrix-shaped parameters of Shampoo (asdl/precondition/shampoo.py:331-339,
 * 351-367). */
int ak_gemm_f32_grouped(int pieces, const int64_t* table, int count, int64_t total_tiles, ak_stream_t stream);

/* y_i <- alpha * M_i x_i for dense row-major [n_i, n_i] fp32 matrices, one launch.  `table` is DEVICE memory,
 * `count` rows of 5 int64: M, x, y (addresses, y not aliasing x), n, first_block, with first_block the running
 * sum of ceil(n/4).  The bias half of Kron.mvp (asdl/symmatrix.py:543-546) for all modules at once. */
/* Largest magnitudes of `count` strided fp32 vectors in one launch (the operand ranges the fp16-piece grouped products
 * scale by).  table: device array of 5 int64 per vector: address, number of elements, element stride (d + 1 walks the
 * diagonal of a [d, d] matrix: for a symmetric positive definite matrix that is its largest magnitude), address of the
 * float word the maximum is folded into (integer atomic maximum on the bit pattern: zero the words first), first block;
 * blocks of ak_absmax_block() elements are numbered in table order, total_blocks of them.  No counterpart in the
 * reference. */
int64_t ak_absmax_block(void);
int ak_absmax_grouped(const int64_t* table, int count, int64_t total_blocks, ak_stream_t stream);

int ak_gemv_f32_grouped(const int64_t* table, int count, int64_t total_blocks, float alpha, ak_stream_t stream);

/* Convolution weight gradients of many modules between the channels-last layout [Cout][kh*kw][Cin] and the
 * contiguous [Cout][Cin][kh*kw] that the Kronecker factors index (to_contiguous != 0: channels-last -> contiguous,
 * else back), one launch.  `table` is DEVICE memory, `count` rows of 5 int64: channels-last address, contiguous
 * address, Cin, kh*kw, first_row (running sum of Cout); total_rows the sum of Cout; Cin*kh*kw at most
 * ak_weight_layout_max_row().  Replaces the .view(B.shape[0], -1) of Kron.mvp (asdl/symmatrix.py:539), which
 * for a channels-last parameter gradient has to gather first. */
int64_t ak_weight_layout_max_row(void);
int ak_weight_layout_grouped(const int64_t* table, int count, int64_t total_rows, int to_contiguous,
                             ak_stream_t stream);

/* G <- grad_scale * Binv G Ainv (G = [dB, dA] in place), bias <- grad_scale * Binv bias when
 * bias != NULL.  ws holds the [dB, dA] intermediate.  Replaces Kron.mvp(use_inv, inplace)
 * (asdl/symmatrix.py:536-548) and the grad_scale pre-multiply of
 * NaturalGradientMaker._precondition_module (asdl/precondition/natural_gradient.py:535-538). */
size_t ak_kron_precond_ws_bytes(int64_t dB, int64_t dA);
int ak_kron_precond(const float* Binv, const float* Ainv, float* G, int64_t dB, int64_t dA,
                    float* bias, float grad_scale, void* ws, size_t ws_bytes, ak_stream_t stream);

/* ak_kron_precond without a workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, serving loops, harnesses that forbid hipMalloc): the [dB, dA] intermediate (and dB floats for the
 * bias) lives in an array of ak_kron_precond_static_max_floats() floats (4 Mi floats = 16 MiB) that is part of the
 * library's device image, one copy per GPU, held until the process ends.  dB*dA + dB beyond that maximum returns
 * AK_ERR_TOO_LARGE and touches nothing.  Calls no hipMalloc / hipFree.  Nothing in the array has to start at zero
 * (both products overwrite their whole output).  All calls on one GPU share the array: calls that may overlap on
 * one GPU (different streams, different threads) race; order them on one stream.  Same results as ak_kron_precond.
 * The first call on a device looks up the array's device address (hipGetSymbolAddress, which may load the library's
 * code object): make it before a stream capture begins.  No counterpart in the reference. */
int64_t ak_kron_precond_static_max_floats(void);

int ak_kron_precond_static(const float* Binv, const float* Ainv, float* G, int64_t dB, int64_t dA,
                           float* bias, float grad_scale, ak_stream_t stream);

/* ---- Shampoo inverse p-th root ---------------------------------------------------- */

/* out_b <- (S_b + r_b I)^(-1/p), r_b = ridge_eps * lambda_max(S_b), for a batch of n x n fp32 statistics
 * (S_b = S + b*strideS, out_b = out + b*strideOut, dense rows): power iteration from the start vectors
 * v0 [batch, n] (the reference draws them from U(-1, 1)), then the coupled Newton iteration.  S_b keeps
 * the ridge on exit, as in the reference.  Convergence tests run on the device: once a matrix's error is
 * below tol, or grows by more than 1.2x (then its previous root is kept), the remaining launches return
 * immediately for it.  stats: device float [batch, 4] = {lambda_max, power iterations, newton iterations,
 * final error}.  n >= 2 (the reference returns the identity for n == 1 without any arithmetic).
 * Statistics of 512 columns and more iterate on 16-bit planes written by the product that makes each matrix
 * (192-wide tiles, n padded to a multiple of 192 in the workspace): two fp16 planes (22 bits of the power-of-two
 * scaled value, three matrix instructions per fp32-grade product) where ridge_eps, p and n bound the root's largest
 * eigenvalue, (ridge_eps (1 + p) / (2 sqrt(n)))^(-1/p), below 4096 and p <= 8; else three bf16 planes (the exact split
 * of the fp32 value, six matrix instructions).  ak_inv_root_plane_format tells which: 0 = fp32 matrices (n < 512),
 * 2, 3.  The environment variable ASDL_AMD_ROOT_FP16_PLANES=0 (read once) keeps every statistic on bf16 planes.
 * ak_inv_root_ws_bytes is 60 bytes per padded element and statistic on planes, 36 per element below that size.
 * Replaces ComputePower / PowerIter / MatPower (asdl/precondition/shampoo.py:465-586). */
size_t ak_inv_root_ws_bytes(int64_t n, int batch);
int ak_inv_root_plane_format(int64_t n, int p, float ridge_eps);
int ak_inv_root_newton(float* S, int64_t n, int batch, int64_t strideS, int p, float ridge_eps,
                       const float* v0, int max_power_iter, float power_tol, int max_iter, float tol,
                       float* out, int64_t strideOut, float* stats, void* ws, size_t ws_bytes,
                       ak_stream_t stream);

/* The same computation in parts, for a host that stops enqueuing once every matrix has converged (the reference's
 * `while error > tol and count < iter_count` of asdl/precondition/shampoo.py:508-521 ends there; the one-call form
 * enqueues max_iter iterations whose kernels exit at once for converged matrices).  `phases` is a bit mask:
 * 1 = power iteration, ridge and start; 2 = `iters` further Newton iterations; 4 = stats.  All parts of one
 * computation get the same arguments and the same workspace, untouched in between.  Between parts the host may read
 * the `batch` int32 words at ws + ak_inv_root_active_offset(n, batch) (after synchronising with the stream): word b is
 * non-zero while matrix b still iterates.  ak_inv_root_newton == phases 7 with iters = max_iter.  `out` holds the
 * roots once the part with bit 4 has run (the last one). */
size_t ak_inv_root_active_offset(int64_t n, int batch);
int ak_inv_root_newton_part(int phases, int iters, float* S, int64_t n, int batch, int64_t strideS, int p,
                            float ridge_eps, const float* v0, int max_power_iter, float power_tol, int max_iter,
                            float tol, float* out, int64_t strideOut, float* stats, void* ws, size_t ws_bytes,
                            ak_stream_t stream);

/* ---- stream helpers (no counterpart in the reference) ------------------------------------ */

/* For hosts that run the statistics kernels on a side stream: events of the HIP runtime this library is linked
 * against, and `after` waits for what `before` holds so far (two runtime calls).  The caller owns the events. */
int ak_event_create(void** event, int timing);
int ak_event_destroy(void* event);
int ak_event_record(void* event, ak_stream_t stream);
int ak_stream_order(ak_stream_t before, ak_stream_t after, void* event);
int ak_event_elapsed_ms(void* start, void* stop, float* ms);

/* ---- measurement aid (no counterpart in the reference) ----------------------------------- */

/* dst <- src, `bytes` bytes (a multiple of 16), by a plain grid-stride kernel: exactly `bytes` read from and `bytes`
 * written to device memory.  The known traffic against which FETCH_SIZE / WRITE_SIZE counter readings of the other
 * kernels are scaled, and the yardstick for the achieved bandwidth of the memory-bound ones. */
int ak_copy_bytes(const void* src, void* dst, int64_t bytes, ak_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif
