/*
 * soap_mi355.h -- C ABI of libsoap_mi355.so: the gfx950 (MI355X) replacement for the SLATE and
 * ELPA pybind11 modules of soap-tp at process_grid_shape == (1, 1).
 *
 * Conventions
 *   - every matrix is dense column-major with a leading dimension (element (i, j) at
 *     p[i + j*ld]) unless a parameter is documented as row-major; this is what a 2-D
 *     block-cyclic buffer degenerates to on a 1x1 process grid;
 *   - all pointers are device pointers owned by the caller; nothing is retained after return;
 *   - `stream` is a hipStream_t (NULL = default stream); calls enqueue work and return without
 *     synchronising;
 *   - `workspace` may be NULL: the library then uses a per-device buffer it grows on demand
 *     (not safe for concurrent use from several streams); otherwise it must hold at least
 *     the bytes reported by the matching *_workspace_bytes query (the sizes do not depend on
 *     soapmi_set_option: they cover both tridiagonalisations and both QR blockings);
 *   - return value 0 = success; <0 = error (SOAPMI_INVALID_ARGUMENT is the analogue of the
 *     std::invalid_argument the reference bindings throw, SOAPMI_RUNTIME_ERROR of
 *     std::runtime_error); soapmi_last_error() returns the message of the calling thread's
 *     most recent failure.
 */
#ifndef SOAP_MI355_H
#define SOAP_MI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SOAPMI_OK 0
#define SOAPMI_INVALID_ARGUMENT (-1)
#define SOAPMI_RUNTIME_ERROR (-2)
#define SOAPMI_NOT_CONVERGED (-3)
#define SOAPMI_WORKSPACE_TOO_SMALL (-4)

/* ---- introspection ------------------------------------------------------------------- */

/* Replaces compiled_gpu_backend() of both reference modules
 * (src/soap_tp/csrc/slate_bindings.cpp:320-323, elpa_bindings.cpp:204-207). Returns "rocm". */
const char* soapmi_compiled_gpu_backend(void);

/* Replaces mpi_world_rank_and_size() (slate_bindings.cpp:324-332, elpa_bindings.cpp:209-217):
 * this library is single-process, so it always reports rank 0 of 1. */
void soapmi_world_rank_and_size(int* rank, int* size);

const char* soapmi_last_error(void);

/* Process-wide tuning knobs (no counterpart in the reference).  Options:
 *   "qr_persistent_max_workgroups"  0..128 (default 128): a QR panel whose grid (rows / 256) fits
 *       runs as one persistent launch whose workgroups exchange partial sums through device memory;
 *       larger panels, or all panels with 0, run one launch per column instead.
 *   "qr_columns_per_round"  1..4 or 32 (default 32): panel columns the persistent QR panel kernel
 *       factors per exchange of partial sums.  The exchange carries the dot products of all the
 *       round's columns; the reflectors after the first follow from those by rank-one corrections
 *       (guarded: a column whose corrected norm shows cancellation ends the round and starts the
 *       next one with directly computed sums); 1 computes every column's sums directly; 32 covers
 *       a whole panel with one exchange of its 32 x 32 Gram matrix, computed on the matrix cores.
 *   "refresh_streams"  1 or 2 (default 2): with 2, soapmi_refresh_f32 runs the left and the right
 *       factorisation chain side by side, the smaller one on a stream the library owns, forked from
 *       and joined back into the caller's stream with events; with 1 everything is enqueued on the
 *       caller's stream, one chain after the other.  The results are the same bit for bit.
 *   "qr_carry_update"  0 or 1 (default 1): with 1, the update of the rest of a 256-column block with a
 *       panel's reflectors rides along in the launch of the next panel (extra workgroups update the
 *       columns behind that panel, the panel's own workgroups update their 32 columns themselves);
 *       with 0 it is a launch of its own between two panels.
 *   "qr_super_block"  0, 256 or 1024 (default 0): the widest compact-WY reflector of the QR.  With
 *       1024 the 256-column blocks are applied only inside a super-block of 1024 columns, and the
 *       matrix beyond it (and the explicit Q) is updated once per super-block by products with
 *       K = 1024; with 256 every block updates the whole trailing matrix (K = 256); 0 takes 1024 up
 *       to n = 4096 and 256 above (the faster one on MI355X by 1 to 4 % either way).  1024 applies
 *       where every panel runs on the whole-panel kernel ("qr_columns_per_round" 32, at most
 *       "qr_persistent_max_workgroups" x 256 rows); other settings use 256.
 *   "persistent_workgroup_budget"  1..256 (default 256): the QR panel kernel and the
 *       tridiagonalisation's column kernel need all workgroups of a launch resident together (one per
 *       256 rows).  The library keeps count of the factorisations that may still be running on a
 *       device and makes a new one wait on the device (stream-wait on an event, no host
 *       synchronisation) for earlier ones until the sum of their workgroup counts fits this budget.
 *       A factorisation larger than the budget runs alone.
 *   "message_spin_limit"  0..4194304 (default 4194304): how many times a workgroup of the QR panel
 *       kernel or of the tridiagonalisation's column kernel polls for another workgroup's message
 *       before it gives up.  Giving up never hangs and never passes silently: the kernels leave,
 *       and the factorisation's output is poisoned with NaN (Q's diagonal, the eigenvalues). */
int soapmi_set_option(const char* name, int64_t value);

/* Failure reporting of the factorisations.  The reference's bindings throw when ELPA or SLATE
 * report an error (src/soap_tp/csrc/elpa_bindings.cpp:77-91,149-171); here a factorisation's
 * kernels are only enqueued when its entry point returns, so a failure found on the device (a
 * persistent kernel that gave up waiting for a message: the output is then NaN-poisoned) is
 * reported afterwards: returns 1 if a factorisation that has finished on the current device
 * since the last call with clear != 0 failed, 0 if none did, <0 on error.  Reads a word of pinned
 * host memory that the device writes: no synchronisation, so it reflects the kernels that have
 * completed so far. */
int soapmi_device_error_flag(int clear);

/* Failure attribution per optimizer state (the reference throws from the failing call itself,
 * src/soap_tp/csrc/elpa_bindings.cpp:77-91,149-171, so its caller knows which state failed).
 * `word` points to one int of device-writable memory that the caller owns and has set to 0 (device
 * memory, or pinned host memory, which the host can then read without synchronising).  While it is
 * set, every factorisation the CALLING THREAD enqueues (soapmi_qr_f32, soapmi_power_iteration_qr_f32,
 * soapmi_refresh_f32, soapmi_eigh_f64/f32, soapmi_initialize_basis_f32) raises *word to 1 instead of
 * the device's word when one of its kernels gives up; NULL restores the per-device word.  The word
 * must stay valid until the kernels enqueued while it was set have finished. */
int soapmi_set_status_word(int* word);

/* ---- Gram preconditioner EMA ---------------------------------------------------------- */

/* P <- lerp(P, G G^T, 1-beta) (side 0, P is rows x rows) or lerp(P, G^T G, 1-beta) (side 1,
 * P is cols x cols).  Replaces the tile loops of
 * update_{left,right}_preconditioner_2d_block_cyclic_ (src/soap_tp/ops/preconditioners.py:678-777,
 * engines :248-408 and :411-623).  G is rows x cols; g_row_major != 0 means element (i, j) is at
 * g[i*ldg + j] (a contiguous torch gradient), otherwise g[i + j*ldg].  Only tiles on or below the
 * diagonal are computed; mirror != 0 also stores the transposed elements so that both
 * triangles of P stay valid (the reference contract, factorizations.py:378). */
int soapmi_gram_ema_f32(const float* g, int64_t rows, int64_t cols, int64_t ldg, int g_row_major, int side,
                        float* p, int64_t ldp, float beta, int mirror, void* stream);

/* Both Gram updates of one step (src/soap_tp/soap.py:425-448: the left and the right update with the
 * same gradient) as one launch: left (rows x rows) <- lerp(left, G G^T, 1-beta) and right
 * (cols x cols) <- lerp(right, G^T G, 1-beta).  Same arithmetic per element as two calls of
 * soapmi_gram_ema_f32; the joint grid fills the compute units better than either product alone. */
int soapmi_gram_ema_pair_f32(const float* g, int64_t rows, int64_t cols, int64_t ldg, int g_row_major, float* left,
                             int64_t ldl, float* right, int64_t ldr, float beta, int mirror, void* stream);

/* Copies the strictly lower triangle of the n x n matrix P onto its upper triangle. */
int soapmi_symmetrize_lower_f32(float* p, int64_t n, int64_t ldp, void* stream);

/* ---- rotations and Adam ---------------------------------------------------------------- */

/* In-place X <- QL^T X QR (forward != 0) or X <- QL X QR^T (forward == 0).  Replaces
 * slate_forward_rotation_float / slate_backward_rotation_float
 * (src/soap_tp/csrc/slate_bindings.cpp:191-315).  Workspace: rows*cols floats. */
int soapmi_rotate_f32(const float* ql, float* x, const float* qr, int64_t rows, int64_t cols, int64_t ldql,
                      int64_t ldx, int64_t ldqr, int forward, void* workspace, size_t workspace_bytes,
                      void* stream);
size_t soapmi_rotate_workspace_bytes(int64_t rows, int64_t cols);

/* Element-wise Adam in the eigenbasis; replaces adam_update (src/soap_tp/ops/optimizer.py:12-44).
 * All four matrices are rows x cols column-major with their own leading dimensions; momentum and
 * variance are updated in place, `update` receives (m/bc1) / (sqrt(v)/sqrt(bc2) + eps). */
int soapmi_adam_f32(const float* gradient, int64_t ldg, float* momentum, int64_t ldm, float* variance,
                    int64_t ldv, float* update, int64_t ldu, int64_t rows, int64_t cols, int64_t step,
                    double beta1, double beta2, double eps, void* stream);

/* The update half of a steady-state step (src/soap_tp/soap.py:327-417 on a 1x1 grid) as four
 * chained products: H = QL^T G ; U = adam(H QR) (moments updated in the product's epilogue, the
 * rotated gradient never reaches memory) ; H = QL U ; update = H QR^T.  `gradient` and `update`
 * are row-major rows x cols (torch-contiguous shards), which absorbs the two layout copies of
 * redistribute_tp_shard_to_2d_block_cyclic / redistribute_2d_block_cyclic_to_tp_shard
 * (optimizer.py:222-392, :64-219).  `eps` is the caller's epsilon; the eps/sqrt(1-beta2^step)
 * rescaling of soap.py:367 is applied inside.  Workspace: 2*rows*cols floats. */
int soapmi_rotate_adam_rotate_f32(const float* gradient, int64_t ldg, float* update, int64_t ldu, const float* ql,
                                  int64_t ldql, const float* qr, int64_t ldqr, float* momentum, int64_t ldm,
                                  float* variance, int64_t ldv, int64_t rows, int64_t cols, int64_t step,
                                  double beta1, double beta2, double eps, void* workspace,
                                  size_t workspace_bytes, void* stream);
size_t soapmi_rotate_adam_rotate_workspace_bytes(int64_t rows, int64_t cols);

/* soapmi_rotate_adam_rotate_f32 for callers that cannot allocate device memory (code under HIP
 * graph capture, serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments without the workspace: the two rows x cols temporaries live in a
 * static device array inside the library (2 x 4194304 floats = 32 MiB per device, held until the
 * process ends), so the call is limited to rows * cols <= 4194304 (2048 x 2048, 1024 x 4096, ...)
 * and returns SOAPMI_INVALID_ARGUMENT beyond that.  It calls no allocation routine; the first
 * call on a device looks up the array's address there.  All calls on one device share the array:
 * calls that overlap in time on one device (different streams or threads) race; calls ordered on
 * one stream do not, and nothing needs clearing between them. */
int soapmi_rotate_adam_rotate_static_f32(const float* gradient, int64_t ldg, float* update, int64_t ldu,
                                         const float* ql, int64_t ldql, const float* qr, int64_t ldqr,
                                         float* momentum, int64_t ldm, float* variance, int64_t ldv, int64_t rows,
                                         int64_t cols, int64_t step, double beta1, double beta2, double eps,
                                         void* stream);

/* Plain product C = alpha*op(A)*op(B) + beta*C on the same kernel the entry points above use;
 * exported for tests and roofline measurement. */
int soapmi_gemm_f32(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha, const float* a,
                    int64_t lda, const float* b, int64_t ldb, float beta, float* c, int64_t ldc, void* stream);
int soapmi_gemm_f64(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, double alpha, const double* a,
                    int64_t lda, const double* b, int64_t ldb, double beta, double* c, int64_t ldc, void* stream);

/* out (rows x cols, column-major, ldo) <- in (row-major, ldi), or the reverse direction.
 * What redistribute_tp_shard_to_2d_block_cyclic / redistribute_2d_block_cyclic_to_tp_shard
 * (optimizer.py:222-392, :64-219) reduce to on one rank. */
int soapmi_row_major_to_col_major_f32(const float* in, int64_t ldi, float* out, int64_t ldo, int64_t rows,
                                      int64_t cols, void* stream);
int soapmi_col_major_to_row_major_f32(const float* in, int64_t ldi, float* out, int64_t ldo, int64_t rows,
                                      int64_t cols, void* stream);

/* ---- basis refresh ------------------------------------------------------------------------ */

/* work <- A Q for the symmetric n x n matrix A (both triangles must be valid).  Replaces
 * slate_symmetric_multiply_float (src/soap_tp/csrc/slate_bindings.cpp:55-123), which on GPU
 * builds is a plain product with the full matrix (:113-116). */
int soapmi_symm_f32(const float* a, const float* q, float* work, int64_t n, int64_t lda, int64_t ldq, int64_t ldw,
                    void* stream);

/* estimates[j] = sum_i q[i, j] * work[i, j]: diag(Q^T P Q) once work = P Q
 * (src/soap_tp/ops/factorizations.py:255-257).  Fixed-order reduction. */
int soapmi_column_dots_f32(const float* q, int64_t ldq, const float* work, int64_t ldw, int64_t rows, int64_t cols,
                           float* estimates, void* stream);

/* order <- argsort(keys, descending) as int64 (factorizations.py:271).  Ties are broken by the
 * smaller index, NaNs sort first (torch's descending order).  Workspace is only used above 16384 keys. */
int soapmi_argsort_desc_f32(const float* keys, int64_t n, int64_t* order, void* workspace, size_t workspace_bytes,
                            void* stream);
size_t soapmi_argsort_workspace_bytes(int64_t n);

/* out[i, j] = in[row_order[i], col_order[j]]; a NULL order is the identity; out must not overlap in. */
int soapmi_gather_f32(const float* in, int64_t ldi, float* out, int64_t ldo, int64_t rows, int64_t cols,
                      const int64_t* row_order, const int64_t* col_order, void* stream);

/* In-place matrix <- matrix[row_order][:, col_order]; replaces permute_2d_block_cyclic_
 * (src/soap_tp/ops/optimizer.py:395-567).  Workspace: rows*cols floats. */
int soapmi_permute_f32(float* matrix, int64_t ld, int64_t rows, int64_t cols, const int64_t* row_order,
                       const int64_t* col_order, void* workspace, size_t workspace_bytes, void* stream);
size_t soapmi_permute_workspace_bytes(int64_t rows, int64_t cols);

/* Returns 1 if order[0..n) is a permutation of range(n), 0 if not, <0 on error
 * (optimizer.py:47-61).  Synchronises the stream.  Workspace: (n + 1) ints. */
int soapmi_is_permutation(const int64_t* order, int64_t n, void* workspace, size_t workspace_bytes, void* stream);

/* Householder QR of the n x n `matrix` (destroyed), explicit orthogonal factor into `q`.
 * Replaces slate_qr_float (src/soap_tp/csrc/slate_bindings.cpp:125-189: geqrf, set Q = I,
 * unmqr); same LAPACK sign convention (diagonal of R opposite in sign to the pivot). */
int soapmi_qr_f32(float* matrix, float* q, int64_t n, int64_t ldmatrix, int64_t ldq, void* workspace,
                  size_t workspace_bytes, void* stream);
size_t soapmi_qr_workspace_bytes(int64_t n);

/* One power iteration and QR for one basis (power_iteration_qr_2d_block_cyclic_,
 * src/soap_tp/ops/factorizations.py:323-360): work = P Q, estimates = column dots,
 * order = argsort(descending), work = work[:, order], Q = qr(work).Q.
 * symmetrize != 0 first copies P's lower triangle onto its upper one (for P maintained by
 * soapmi_gram_ema_f32 with mirror == 0).  `estimates` may be NULL. */
int soapmi_power_iteration_qr_f32(float* p, float* q, float* work, int64_t n, int64_t ldp, int64_t ldq,
                                  int64_t ldw, int symmetrize, int64_t* order, float* estimates, void* workspace,
                                  size_t workspace_bytes, void* stream);
size_t soapmi_power_iteration_qr_workspace_bytes(int64_t n);

/* refresh_bases_and_transport_optimizer_state_ (src/soap_tp/ops/factorizations.py:550-614):
 * momentum to parameter space with the old bases, power iteration + QR on both sides, variance
 * <- variance[left_order][:, right_order], momentum into the new bases.
 * The two sides' factorisations run side by side: the smaller one is enqueued on a second stream
 * that the library keeps per device (default priority), forked from `stream` and joined back into
 * it with events, so for the caller all work is still ordered on `stream`. */
int soapmi_refresh_f32(float* momentum, int64_t ldm, float* variance, int64_t ldv, float* left_preconditioner,
                       int64_t ldl, float* right_preconditioner, int64_t ldr, float* q_left, int64_t ldql,
                       float* q_right, int64_t ldqr, float* left_work, int64_t ldlw, float* right_work,
                       int64_t ldrw, int64_t rows, int64_t cols, int symmetrize, int64_t* left_order,
                       int64_t* right_order, void* workspace, size_t workspace_bytes, void* stream);
size_t soapmi_refresh_workspace_bytes(int64_t rows, int64_t cols);

/* ---- symmetric eigensolver (basis initialisation) ------------------------------------------ */

/* All eigenpairs of the symmetric n x n matrix `a` (lower triangle referenced, contents
 * destroyed): eigenvalues ascending into `eigenvalues`, eigenvectors into the columns of `q`.
 * Replaces elpa_eigenvectors_2d_block_cyclic_double / initialize_basis_2d_block_cyclic_ of the
 * ELPA module (src/soap_tp/csrc/elpa_bindings.cpp:61-196, alias :234-235; one-stage solver, nev = n,
 * ascending, input destroyed) on a 1x1 grid, where local_rows == lda == n.  Householder
 * tridiagonalisation, divide and conquer, back-transformation; no host synchronisation. */
int soapmi_eigh_f64(double* a, double* eigenvalues, double* q, int64_t n, int64_t lda, int64_t ldq,
                    void* workspace, size_t workspace_bytes, void* stream);
int soapmi_eigh_f32(float* a, float* eigenvalues, float* q, int64_t n, int64_t lda, int64_t ldq, void* workspace,
                    size_t workspace_bytes, void* stream);
size_t soapmi_eigh_workspace_bytes(int64_t n, int element_bytes);

/* Descending eigenbasis of the preconditioner P into Q, eigenvalues (descending, float) into
 * `eigenvalues`: initialize_basis_2d_block_cyclic_ (src/soap_tp/ops/factorizations.py:363-547) on a
 * 1x1 grid.  implementation 0 ("elpa", :472-547): work <- -P, float64 copies, ascending solve of
 * -P, Q = float(Q64), eigenvalues = -lambda.  implementation 1 ("eigh", :421-470): float32 solve
 * of P + 1e-30 I, columns and eigenvalues flipped.  Only the lower triangle of P is read. */
int soapmi_initialize_basis_f32(const float* p, float* q, float* work, float* eigenvalues, int64_t n, int64_t ldp,
                                int64_t ldq, int64_t ldw, int implementation, void* workspace,
                                size_t workspace_bytes, void* stream);
size_t soapmi_initialize_basis_workspace_bytes(int64_t n, int implementation);

#ifdef __cplusplus
}
#endif
#endif /* SOAP_MI355_H */
