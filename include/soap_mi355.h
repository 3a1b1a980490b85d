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
 *     the bytes reported by the matching *_workspace_bytes query;
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

#ifdef __cplusplus
}
#endif
#endif /* SOAP_MI355_H */
