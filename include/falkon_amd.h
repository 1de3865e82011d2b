/*
 * falkon_amd -- C ABI of the MI355X (gfx950) Gaussian kernel-vector products.
 *
 * Every entry point is plain C: device pointers, sizes, element strides and a
 * HIP stream handle (passed as void*).  No torch types cross this boundary.
 * All functions return 0 on success or a negative FLK_E* code; the message of
 * the last failure on the calling thread is available from flk_last_error().
 * Nothing here synchronises the device or allocates device memory: work is
 * enqueued on `stream`, scratch space comes from the caller (`workspace`).
 *
 * Matrices are described as (pointer, rows, cols, row_stride, col_stride) with
 * strides in ELEMENTS, so both C-ordered (col_stride == 1) and Fortran-ordered
 * (row_stride == 1) operands of the reference are accepted as they are
 * (falkon/mmv_ops/utils.py:36-39 requires only that some stride equals one).
 *
 * dtype: FLK_F32 (0) or FLK_F64 (1); all operands of a call share it
 * (falkon/kernels/kernel.py:78-79,102-103).  FLK_F32_BF16X3 (2), accepted by the fmmv / fdmmv / fmm entry
 * points and their workspace queries only (fmm: beyond 64 features and without compute_f64; otherwise as FLK_F32), is fp32 data and fp32 results with the cross term x.c of the
 * squared distance formed on the bfloat16 matrix cores: every scaled fp32 value is split exactly into
 * three bfloat16 pieces (3 x 8 = 24 significant bits) and six partial products are accumulated in fp32,
 * which keeps the accuracy of the fp32 dot product (measured: the same distance from the fp64 result as
 * FLK_F32) at 16 features per matrix instruction instead of 2.  It has no counterpart in the reference.  Where
 * the fp32 MFMA kernels are the faster route (5 to 8 right-hand sides at d <= 32, more than 16 at d <= 62) they serve this code too.
 */
#ifndef FALKON_AMD_H
#define FALKON_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FLK_F32 0
#define FLK_F64 1
#define FLK_F32_BF16X3 2

/* Radial kernels K(x, c) = f(D), D = |x/sigma - c/sigma| (falkon/kernels/distance_kernel.py):
 * Gaussian exp(-D^2/2) (:140-159), Laplacian exp(-D) (:182-205), Matern nu = 3/2 and 5/2 (:225-269;
 * nu = 1/2 is the Laplacian, nu = inf the Gaussian, :235-238).  The flk_gauss_* entry points are the
 * flk_kernel_* ones with FLK_GAUSSIAN.
 * FLK_LAPLACIAN_DU is exp(-D)/D, and 0 where D^2 <= 1e-20: up to the factor -1/2 the derivative of the
 * Laplacian with respect to D^2, zero where the reference's clamp of D^2 (:100) cuts the gradient.  The
 * derivatives of the other three are multiples of kernels already in the list (Gaussian: -1/2 itself;
 * Matern 3/2: -3/2 Laplacian with sigma/sqrt(3); Matern 5/2: -5/6 Matern 3/2 with sigma*sqrt(3/5)), so
 * these five cover the backward pass of the kernel-vector product (falkon/mmv_ops/fmmv.py:405-485). */
#define FLK_GAUSSIAN  0
#define FLK_LAPLACIAN 1
#define FLK_MATERN32  2
#define FLK_MATERN52  3
#define FLK_LAPLACIAN_DU 4

#define FLK_OK          0
#define FLK_EINVAL     -1   /* bad argument (shape, stride, dtype, null pointer)      */
#define FLK_ENOMEM     -2   /* workspace too small                                    */
#define FLK_EUNSUPPORTED -3 /* shape outside what the compiled kernels cover          */
#define FLK_EHIP       -4   /* a HIP runtime call or kernel launch failed             */

/* Library version (major*10000 + minor*100 + patch). */
int flk_version(void);

/* Message describing the last non-zero return on this thread ("" if none). */
const char *flk_last_error(void);

/* Largest feature dimension and number of right-hand sides the kernels cover: calls beyond them return
 * FLK_EUNSUPPORTED, and the size queries below return 0 for them, as for a negative shape or an unknown dtype. */
int64_t flk_max_d(int dtype);
int64_t flk_max_t(void);

/* Instrumentation (no counterpart in the reference, which times whole calls with
 * falkon/utils/tictoc.py:19-63): when enabled, the library brackets every launch of the
 * product kernel with HIP events on the launch stream.  flk_kernel_timing_read waits for
 * the recorded events, returns the summed kernel time and the number of launches since
 * the last read/enable, and clears the records. */
int flk_kernel_timing_enable(int on);
int flk_kernel_timing_read(double *total_ms, int64_t *launches);

/* ---- packed operands ------------------------------------------------------
 * The kernels consume each data matrix in a "packed" form: rows are scaled by
 * a kernel-specific factor over sigma (sqrt(log2 e) for the Gaussian in f32, sqrt(2048 log2 e) in f64: a packed
 * operand is only valid for the kernel and the dtype it was packed for), regrouped in blocks of 32 (f32) or 16 (f64) rows stored
 * feature-major, zero padded, and followed by the vector -1/2*||row||^2.
 * This replaces the reference's per-block `mat / sigma` and `square_norm`
 * prologue of rbf_core (falkon/kernels/distance_kernel.py:148-154;
 * falkon/c_ext/ops/cuda/cuda_square_norm.cu:15-68).
 */

/* Bytes needed for the packed form of an n x d matrix. */
size_t flk_gauss_packed_bytes(int64_t n, int64_t d, int dtype);

/* Pack X[n,d].  sigma is a DEVICE array of n_sigma (1 or d) lengthscales in the
 * data dtype (the reference moves sigma to the data's device and dtype,
 * distance_kernel.py:148).  Any other n_sigma is FLK_EINVAL, which the host
 * layer turns into the RuntimeError the reference raises
 * (falkon/tests/test_kernels.py:338-358). */
int flk_gauss_pack(const void *X, int64_t n, int64_t d, int64_t x_rs, int64_t x_cs,
                   const void *sigma, int64_t n_sigma, int dtype,
                   void *packed, size_t packed_bytes, void *stream);

/* ---- products on packed operands -------------------------------------------
 * out[b,t] = sum_a K(A_a, B_b) * vec[a,t]  (+ addend[b,t] if addend != NULL)
 * with A = n_a packed rows (the reduction side) and B = n_b packed rows (the
 * output side).  K(X1,X2) @ v is (A=X2, B=X1, vec=v); K(X1,X2)^T @ u is
 * (A=X1, B=X2, vec=u).  out is overwritten, never accumulated into
 * (falkon/mmv_ops/fmmv.py:369,732).
 */
size_t flk_gauss_mmv_packed_workspace_bytes(int64_t n_a, int64_t n_b, int64_t d, int64_t t, int dtype);

int flk_gauss_mmv_packed(const void *packed_a, int64_t n_a, const void *packed_b, int64_t n_b, int64_t d,
                         const void *vec, int64_t vec_rs, int64_t vec_cs, int64_t t,
                         const void *addend, int64_t add_rs, int64_t add_cs,
                         void *out, int64_t out_rs, int64_t out_cs, int dtype,
                         void *workspace, size_t workspace_bytes, void *stream);

/* ---- one-call products on plain matrices ----------------------------------
 * flk_gauss_fmmv  replaces falkon.mmv_ops.fmmv.fmmv for the dense Gaussian case
 *   (falkon/mmv_ops/fmmv.py:960-973 -> :309-402 -> distance_kernel.py:140-159):
 *   out[n,t] = K(X1[n,d], X2[m,d]) @ v[m,t].
 * flk_gauss_fdmmv replaces falkon.mmv_ops.fmmv.fdmmv
 *   (falkon/mmv_ops/fmmv.py:976-1131 -> :683-767):
 *   out[m,t] = K^T @ (K @ v + w), v[m,t] required, w[n,t] may be NULL.
 * Both pack X1 and X2 into the workspace, never materialise K, and leave the
 * inputs untouched.  The workspace must hold at least the number of bytes the
 * matching *_workspace_bytes call returns.
 * A NaN or an infinity in a row of X1 or X2 gives NaN in every result that row
 * enters, as in the reference (falkon/kernels/distance_kernel.py:88-101), although
 * the kernels clamp the kernel value: the rows' half norms carry the information.
 */
size_t flk_gauss_fmmv_workspace_bytes(int64_t n, int64_t m, int64_t d, int64_t t, int dtype);

int flk_gauss_fmmv(const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs,
                   const void *X2, int64_t m, int64_t x2_rs, int64_t x2_cs, int64_t d,
                   const void *sigma, int64_t n_sigma,
                   const void *v, int64_t v_rs, int64_t v_cs, int64_t t,
                   void *out, int64_t out_rs, int64_t out_cs, int dtype,
                   void *workspace, size_t workspace_bytes, void *stream);

size_t flk_gauss_fdmmv_workspace_bytes(int64_t n, int64_t m, int64_t d, int64_t t, int dtype);

int flk_gauss_fdmmv(const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs,
                    const void *X2, int64_t m, int64_t x2_rs, int64_t x2_cs, int64_t d,
                    const void *sigma, int64_t n_sigma,
                    const void *v, int64_t v_rs, int64_t v_cs,
                    const void *w, int64_t w_rs, int64_t w_cs, int64_t t,
                    void *out, int64_t out_rs, int64_t out_cs, int dtype,
                    void *workspace, size_t workspace_bytes, void *stream);

/* ---- fdmmv for callers that cannot allocate ---------------------------------
 * flk_gauss_fdmmv_noalloc has no counterpart in the reference.  It is flk_gauss_fdmmv without the workspace
 * argument, for callers that cannot obtain device memory at the call: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  The workspace is an array of FLK_NOALLOC_SCRATCH_BYTES
 * bytes that is part of the library's device code: every GPU on which the library's device code is loaded (by the
 * first flk_* call of any kind that launches there) holds its own copy from then until the process ends, whether
 * or not this entry point is ever called.  The array's device address is looked up on the first call of this entry
 * point on a GPU: make that first call outside a graph capture (the tests capture after one eager call).
 * The call allocates and frees nothing and enqueues the same kernels
 * as flk_gauss_fdmmv, so the results are bit-identical to it.  A problem whose
 * flk_gauss_fdmmv_workspace_bytes(n, m, d, t, dtype) exceeds FLK_NOALLOC_SCRATCH_BYTES is refused with
 * FLK_ENOMEM and a message naming both sizes.  All calls on one GPU share that GPU's array: two calls whose
 * kernels overlap in time (different streams, different threads) race on it, so keep them on one stream or
 * order them yourself.  The array keeps the previous call's contents; every call writes what it reads. */
#define FLK_NOALLOC_SCRATCH_BYTES (64u << 20)

int flk_gauss_fdmmv_noalloc(const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs,
                            const void *X2, int64_t m, int64_t x2_rs, int64_t x2_cs, int64_t d,
                            const void *sigma, int64_t n_sigma,
                            const void *v, int64_t v_rs, int64_t v_cs,
                            const void *w, int64_t w_rs, int64_t w_cs, int64_t t,
                            void *out, int64_t out_rs, int64_t out_cs, int dtype, void *stream);

/* ---- conjugate-gradient iteration on device scalars ---------------------------
 * flk_cg_update replaces the vector work of one iteration of the reference's multi-right-hand-side solver
 * (falkon/optim/conjgrad.py:125-163: alpha = rsold / (sum(P * AP) + eps); X += P alpha; R -= AP alpha (or
 * R = B - A X every cg_full_gradient_every iterations); rsnew = sum(R^2); converged = rsnew < tol^2, stop when
 * every column has; P = R + P rsnew / (rsold + eps)), one workgroup per right-hand side, with the step lengths,
 * residual norms and convergence flags kept on the device, so that the host need not wait for an iteration
 * before it enqueues the next.  X, R, P, Q, B are m x t with the same element strides (rs, cs), one of them 1.
 *   mode 0: whole iteration, Q = A P.
 *   mode 1: step length and X += P alpha only, Q = A P; then, with Q = A X,
 *   mode 2: R = B - Q and the rest of the iteration (the reference's full-gradient iterations, :133-138).
 * rsold: t squared residual norms in the data dtype, set by the caller to sum(R^2) before the first iteration.
 * state: flk_cg_state_ints(t) int32, zeroed by the caller before the first iteration: [0] becomes 1 once every
 *   column has converged, and every later call then leaves X, R, P untouched (the reference's break, :143-145);
 *   [1] counts the iterations applied; [2 .. 2+2t) are the columns' convergence flags of the last two iterations;
 *   [2+2t .. 2+3t) marks columns that left the solve (differential != 0: a converged column is frozen at its
 *   value, the reference's cg_differential_convergence, :113-161).
 * iteration: index of the iteration (its parity selects the flag buffer); mode 1 and mode 2 of one iteration pass
 *   the same value.  Sums are taken in a fixed order in double precision: results are reproducible. */
int64_t flk_cg_state_ints(int64_t t);

int flk_cg_update(int mode, void *X, void *R, void *P, const void *Q, const void *B, int64_t m, int64_t t,
                  int64_t rs, int64_t cs, void *rsold, int32_t *state, int64_t iteration,
                  double eps, double tol2, int differential, int dtype, void *stream);

/* ---- triangular solves of the preconditioner ----------------------------------
 * flk_tri_solve replaces the triangular solves with the preconditioner's two Cholesky factors that every
 * conjugate-gradient iteration performs (falkon/preconditioner/flk_preconditioner.py:166-256: invA, invAt, invT,
 * invTt, there the library's trsm; falkon/optim/conjgrad.py:242-256 is the caller) for 1 .. 4 right-hand sides.
 *   L: m x m lower-triangular factor, element (i, j) at L[i*ld + j] (row_major != 0) or L[i + j*ld]; only the
 *      part below the diagonal blocks is read.
 *   dinv, dinv_t: inverses of the diagonal blocks L[k*block .. , k*block ..] and the transposes of those inverses,
 *      block k at + k*block*block elements, row-major with leading dimension `block` (a smaller last block keeps
 *      that leading dimension); the caller computes them once per factor.  The inverses are triangular, and the
 *      kernels read a few entries on the other side of the diagonal (rows are processed four at a time): those
 *      entries must be stored as zeros.  block: a multiple of 4.
 *   transposed == 0 solves L x = b, otherwise L^T x = b.
 *   b, x: t columns of m elements each, column c at + c*ldb, + c*ldx; work: flk_tri_solve_work_elems(m, t, block)
 *      elements of the data dtype (partial sums of the panel products); three distinct buffers.
 * A solve reads the triangle once (two launches per diagonal block: a panel product over long contiguous rows and
 * the product with the inverted block), sums in a fixed order in double precision (reproducible), takes no
 * workspace beyond `work` and does not synchronise. */
int64_t flk_tri_solve_work_elems(int64_t m, int64_t t, int64_t block);

int flk_tri_solve(int dtype, int transposed, const void *L, int64_t m, int64_t ld, int row_major,
                  const void *dinv, const void *dinv_t, int64_t block,
                  const void *b, int64_t ldb, void *x, int64_t ldx, int64_t t, void *work, void *stream);

/* ---- diagonal tiles of the preconditioner's Cholesky factorisations ---------------
 * flk_potrf_tile serves the two factorisations of M x M matrices that build the preconditioner
 * (falkon/preconditioner/flk_preconditioner.py:115,152: potrf_wrapper; falkon/preconditioner/pc_utils.py: the
 * library potrf behind it).  A blocked factorisation spends nearly all its flop in matrix products, but its diagonal
 * tiles are a chain of M dependent column steps; this entry point runs that chain for one tile inside one workgroup.
 *   A: n x n, n <= flk_potrf_tile_rows(dtype), element (i, j) at A[i*lda + j]; the lower triangle is read and
 *      overwritten with the Cholesky factor L (A = L L^T); the elements above the diagonal are left alone.
 *   inv: n x n at inv[i*ldinv + j], a buffer distinct from A: receives L^-1 with zeros above the diagonal, so that the
 *      triangular solve of the panel below the tile is the matrix product  panel <- panel * inv^T.
 *   info: one int in device memory that the caller clears before the first tile.  A pivot that is not positive (or
 *      is NaN) at row j stores info_base + j + 1 there unless a failure is already recorded; L and inv are NaN from
 *      that row on.  The call does not synchronise and does not read info on the host. */
int64_t flk_potrf_tile_rows(int dtype);

int flk_potrf_tile(int dtype, void *A, int64_t n, int64_t lda, void *inv, int64_t ldinv, int *info, int64_t info_base,
                   void *stream);

/* ---- explicit kernel matrix -------------------------------------------------
 * flk_gauss_fmm replaces falkon.mmv_ops.fmm.fmm for the dense Gaussian case
 *   (falkon/mmv_ops/fmm.py:699-708 -> :298-388 block loop -> distance_kernel.py:140-159):
 *   out[n,m] = K(X1[n,d], X2[m,d]), overwritten.  out needs a unit stride in
 *   one of its two dimensions (falkon/mmv_ops/utils.py:36-39).
 * compute_f64 != 0 with dtype = FLK_F32 evaluates the kernel in double
 *   precision on the single-precision data and rounds the result once, the
 *   reference's `no_single_kernel` rule for the preconditioner's K(C,C)
 *   (falkon/mmv_ops/fmm.py:619-622); it is ignored for dtype = FLK_F64.
 */
size_t flk_gauss_fmm_workspace_bytes(int64_t n, int64_t m, int64_t d, int dtype, int compute_f64);

int flk_gauss_fmm(const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs,
                  const void *X2, int64_t m, int64_t x2_rs, int64_t x2_cs, int64_t d,
                  const void *sigma, int64_t n_sigma,
                  void *out, int64_t out_rs, int64_t out_cs, int dtype, int compute_f64,
                  void *workspace, size_t workspace_bytes, void *stream);

/* ---- the same entry points for any of the radial kernels ----------------------
 * `kernel` is one of FLK_GAUSSIAN / FLK_LAPLACIAN / FLK_MATERN32 / FLK_MATERN52 / FLK_LAPLACIAN_DU; everything else as in
 * the flk_gauss_* function of the same name, whose *_workspace_bytes / flk_gauss_packed_bytes sizes
 * apply to every kernel.  Packed operands are specific to the kernel they were packed for (the
 * Gaussian rows carry an extra factor).  These replace fmmv / fdmmv / fmm for the reference's
 * LaplacianKernel and MaternKernel (falkon/kernels/distance_kernel.py:434-648).
 */
int flk_kernel_pack(int kernel, const void *X, int64_t n, int64_t d, int64_t x_rs, int64_t x_cs,
                    const void *sigma, int64_t n_sigma, int dtype,
                    void *packed, size_t packed_bytes, void *stream);

int flk_kernel_mmv_packed(int kernel, const void *packed_a, int64_t n_a, const void *packed_b, int64_t n_b, int64_t d,
                          const void *vec, int64_t vec_rs, int64_t vec_cs, int64_t t,
                          const void *addend, int64_t add_rs, int64_t add_cs,
                          void *out, int64_t out_rs, int64_t out_cs, int dtype,
                          void *workspace, size_t workspace_bytes, void *stream);

int flk_kernel_fmmv(int kernel, const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs,
                    const void *X2, int64_t m, int64_t x2_rs, int64_t x2_cs, int64_t d,
                    const void *sigma, int64_t n_sigma,
                    const void *v, int64_t v_rs, int64_t v_cs, int64_t t,
                    void *out, int64_t out_rs, int64_t out_cs, int dtype,
                    void *workspace, size_t workspace_bytes, void *stream);

int flk_kernel_fdmmv(int kernel, const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs,
                     const void *X2, int64_t m, int64_t x2_rs, int64_t x2_cs, int64_t d,
                     const void *sigma, int64_t n_sigma,
                     const void *v, int64_t v_rs, int64_t v_cs,
                     const void *w, int64_t w_rs, int64_t w_cs, int64_t t,
                     void *out, int64_t out_rs, int64_t out_cs, int dtype,
                     void *workspace, size_t workspace_bytes, void *stream);

int flk_kernel_fmm(int kernel, const void *X1, int64_t n, int64_t x1_rs, int64_t x1_cs,
                   const void *X2, int64_t m, int64_t x2_rs, int64_t x2_cs, int64_t d,
                   const void *sigma, int64_t n_sigma,
                   void *out, int64_t out_rs, int64_t out_cs, int dtype, int compute_f64,
                   void *workspace, size_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FALKON_AMD_H */
