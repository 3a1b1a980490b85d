// extern "C" surface of libsoap_mi355.so (declared in include/soap_mi355.h).
#include <stdarg.h>

#include <mutex>

#include "../../include/soap_mi355.h"
#include "common.hpp"
#include "elementwise.hpp"
#include "gemm.hpp"

namespace soapmi {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
const char* last_error() { return g_error; }

// Per-device grow-only scratch used when the caller passes no workspace.
struct InternalScratch {
  void* ptr = nullptr;
  size_t size = 0;
};
static InternalScratch g_scratch[64];
static std::mutex g_scratch_mutex;

static int resolve_workspace(void* user, size_t user_bytes, size_t need, void** out) {
  if (user != nullptr) {
    if (user_bytes < need) {
      set_error("workspace holds %zu bytes, %zu are required", user_bytes, need);
      return kWorkspaceTooSmall;
    }
    *out = user;
    return kOk;
  }
  int dev = 0;
  SOAPMI_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) {
    set_error("unsupported device index %d", dev);
    return kRuntimeError;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  InternalScratch& s = g_scratch[dev];
  if (s.size < need) {
    if (s.ptr) {
      SOAPMI_HIP(hipDeviceSynchronize());
      SOAPMI_HIP(hipFree(s.ptr));
      s.ptr = nullptr;
      s.size = 0;
    }
    SOAPMI_HIP(hipMalloc(&s.ptr, need));
    s.size = need;
  }
  *out = s.ptr;
  return kOk;
}

static AdamScalars make_adam_scalars(int64_t step, double beta1, double beta2, double eps_in) {
  AdamScalars s;
  s.beta1 = (float)beta1;
  s.beta2 = (float)beta2;
  s.one_minus_beta1 = (float)(1.0 - beta1);
  s.one_minus_beta2 = (float)(1.0 - beta2);
  s.bias_correction1 = (float)(1.0 - pow(beta1, (double)step));
  s.sqrt_bias_correction2 = (float)sqrt(1.0 - pow(beta2, (double)step));
  s.eps = (float)eps_in;
  return s;
}

static int check_adam_args(int64_t step, double beta1, double beta2, double eps) {
  SOAPMI_REQUIRE(step >= 1, "step must be positive, got %lld.", (long long)step);
  SOAPMI_REQUIRE(beta1 >= 0.0 && beta1 < 1.0, "beta1 must be in [0, 1), got %g.", beta1);
  SOAPMI_REQUIRE(beta2 >= 0.0 && beta2 < 1.0, "beta2 must be in [0, 1), got %g.", beta2);
  SOAPMI_REQUIRE(eps > 0.0, "eps must be positive, got %g.", eps);
  return kOk;
}

}  // namespace soapmi

using namespace soapmi;

extern "C" {

const char* soapmi_compiled_gpu_backend(void) { return "rocm"; }

void soapmi_world_rank_and_size(int* rank, int* size) {
  if (rank) *rank = 0;
  if (size) *size = 1;
}

const char* soapmi_last_error(void) { return last_error(); }

int soapmi_gemm_f32(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha, const float* a,
                    int64_t lda, const float* b, int64_t ldb, float beta, float* c, int64_t ldc, void* stream) {
  SOAPMI_REQUIRE(m >= 0 && n >= 0 && k >= 0, "matrix dimensions must be non-negative");
  SOAPMI_REQUIRE(a && b && c, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(lda >= (trans_a ? k : m) && ldb >= (trans_b ? n : k) && ldc >= m && lda > 0 && ldb > 0 && ldc > 0,
                 "leading dimensions are too small");
  return gemm<float>((hipStream_t)stream, trans_a, trans_b, (int)m, (int)n, (int)k, alpha, a, lda, b, ldb, beta, c,
                     ldc);
}

int soapmi_gemm_f64(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, double alpha, const double* a,
                    int64_t lda, const double* b, int64_t ldb, double beta, double* c, int64_t ldc, void* stream) {
  SOAPMI_REQUIRE(m >= 0 && n >= 0 && k >= 0, "matrix dimensions must be non-negative");
  SOAPMI_REQUIRE(a && b && c, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(lda >= (trans_a ? k : m) && ldb >= (trans_b ? n : k) && ldc >= m && lda > 0 && ldb > 0 && ldc > 0,
                 "leading dimensions are too small");
  return gemm<double>((hipStream_t)stream, trans_a, trans_b, (int)m, (int)n, (int)k, alpha, a, lda, b, ldb, beta,
                      c, ldc);
}

int soapmi_gram_ema_f32(const float* g, int64_t rows, int64_t cols, int64_t ldg, int g_row_major, int side,
                        float* p, int64_t ldp, float beta, int mirror, void* stream) {
  SOAPMI_REQUIRE(g && p, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(rows >= 0 && cols >= 0, "matrix dimensions must be non-negative");
  SOAPMI_REQUIRE(side == 0 || side == 1, "side must be 0 (left) or 1 (right), got %d.", side);
  SOAPMI_REQUIRE(beta >= 0.0f && beta <= 1.0f, "beta must be in [0, 1], got %g.", (double)beta);
  SOAPMI_REQUIRE(ldg >= (g_row_major ? cols : rows) && ldg > 0, "gradient leading dimension is too small");
  const int64_t n = side == 0 ? rows : cols;
  const int64_t k = side == 0 ? cols : rows;
  SOAPMI_REQUIRE(ldp >= n && ldp > 0, "preconditioner leading dimension is too small");
  if (n == 0) return kOk;
  // Stored matrix S (column-major, ld = ldg): row-major G is S = G^T (cols x rows).
  // left  = G G^T : row-major -> S^T S (transA=1, transB=0) ; col-major -> S S^T (0, 1)
  // right = G^T G : row-major -> S S^T (0, 1)               ; col-major -> S^T S (1, 0)
  const bool stts = (side == 0) == (g_row_major != 0);
  const int ta = stts ? 1 : 0, tb = stts ? 0 : 1;
  GemmProblem<float> prob = make_problem<float>(ta, tb, (int)n, (int)n, (int)k, g, ldg, g, ldg, true);
  EpiEmaLower<float> epi{p, ldp, 1.0f - beta, mirror};
  return launch_gemm<float>((hipStream_t)stream, prob, epi, 1);
}

int soapmi_symmetrize_lower_f32(float* p, int64_t n, int64_t ldp, void* stream) {
  SOAPMI_REQUIRE(p, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(n >= 0 && ldp >= n && ldp > 0, "invalid matrix size or leading dimension");
  if (n == 0) return kOk;
  unsigned nb = (unsigned)ceil_div64(n, 64);
  hipLaunchKernelGGL((symmetrize_lower_kernel<float>), dim3(nb, nb), dim3(256), 0, (hipStream_t)stream, p, ldp,
                     (int)n);
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

size_t soapmi_rotate_workspace_bytes(int64_t rows, int64_t cols) {
  WorkspaceSizer w;
  w.take<float>((size_t)rows * cols);
  return w.total();
}

int soapmi_rotate_f32(const float* ql, float* x, const float* qr, int64_t rows, int64_t cols, int64_t ldql,
                      int64_t ldx, int64_t ldqr, int forward, void* workspace, size_t workspace_bytes,
                      void* stream) {
  SOAPMI_REQUIRE(ql && x && qr, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(rows > 0 && cols > 0 && ldql > 0 && ldx > 0 && ldqr > 0,
                 "matrix dimensions and leading dimensions must be positive");
  SOAPMI_REQUIRE(ldql >= rows && ldx >= rows && ldqr >= cols, "leading dimensions are too small");
  void* ws = nullptr;
  int rc = resolve_workspace(workspace, workspace_bytes, soapmi_rotate_workspace_bytes(rows, cols), &ws);
  if (rc) return rc;
  Workspace w(ws, soapmi_rotate_workspace_bytes(rows, cols));
  float* h = w.take<float>((size_t)rows * cols);
  hipStream_t s = (hipStream_t)stream;
  const int m = (int)rows, n = (int)cols;
  // forward : H = QL^T X ; X = H QR        backward : H = QL X ; X = H QR^T
  rc = gemm<float>(s, forward ? 1 : 0, 0, m, n, m, 1.0f, ql, ldql, x, ldx, 0.0f, h, rows);
  if (rc) return rc;
  return gemm<float>(s, 0, forward ? 0 : 1, m, n, n, 1.0f, h, rows, qr, ldqr, 0.0f, x, ldx);
}

int soapmi_adam_f32(const float* gradient, int64_t ldg, float* momentum, int64_t ldm, float* variance,
                    int64_t ldv, float* update, int64_t ldu, int64_t rows, int64_t cols, int64_t step,
                    double beta1, double beta2, double eps, void* stream) {
  int rc = check_adam_args(step, beta1, beta2, eps);
  if (rc) return rc;
  SOAPMI_REQUIRE(rows >= 0 && cols >= 0, "matrix dimensions must be non-negative");
  if (rows == 0 || cols == 0) return kOk;
  SOAPMI_REQUIRE(gradient && momentum && variance && update, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(ldg >= rows && ldm >= rows && ldv >= rows && ldu >= rows, "leading dimensions are too small");
  AdamScalars sc = make_adam_scalars(step, beta1, beta2, eps);
  unsigned gy = (unsigned)(cols < 4096 ? cols : 4096);
  hipLaunchKernelGGL(adam_kernel, dim3((unsigned)ceil_div64(rows, 256), gy), dim3(256), 0, (hipStream_t)stream,
                     gradient, ldg, momentum, ldm, variance, ldv, update, ldu, (int)rows, (int)cols, sc);
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

size_t soapmi_rotate_adam_rotate_workspace_bytes(int64_t rows, int64_t cols) {
  WorkspaceSizer w;
  w.take<float>((size_t)rows * cols);
  w.take<float>((size_t)rows * cols);
  return w.total();
}

int soapmi_rotate_adam_rotate_f32(const float* gradient, int64_t ldg, float* update, int64_t ldu, const float* ql,
                                  int64_t ldql, const float* qr, int64_t ldqr, float* momentum, int64_t ldm,
                                  float* variance, int64_t ldv, int64_t rows, int64_t cols, int64_t step,
                                  double beta1, double beta2, double eps, void* workspace,
                                  size_t workspace_bytes, void* stream) {
  int rc = check_adam_args(step, beta1, beta2, eps);
  if (rc) return rc;
  SOAPMI_REQUIRE(gradient && update && ql && qr && momentum && variance, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(rows > 0 && cols > 0, "matrix dimensions must be positive");
  SOAPMI_REQUIRE(ldg >= cols && ldu >= cols, "row-major leading dimensions are too small");
  SOAPMI_REQUIRE(ldql >= rows && ldqr >= cols && ldm >= rows && ldv >= rows, "leading dimensions are too small");
  const size_t need = soapmi_rotate_adam_rotate_workspace_bytes(rows, cols);
  void* ws = nullptr;
  rc = resolve_workspace(workspace, workspace_bytes, need, &ws);
  if (rc) return rc;
  Workspace w(ws, need);
  float* h = w.take<float>((size_t)rows * cols);
  float* u = w.take<float>((size_t)rows * cols);
  hipStream_t s = (hipStream_t)stream;
  const int m = (int)rows, n = (int)cols;
  const double bc2 = 1.0 - pow(beta2, (double)step);
  AdamScalars sc = make_adam_scalars(step, beta1, beta2, eps / sqrt(bc2));

  // 1. H = QL^T G.  The row-major gradient is the column-major matrix S = G^T (cols x rows, ld ldg),
  //    so op(B) = S^T.
  rc = gemm<float>(s, 1, 1, m, n, m, 1.0f, ql, ldql, gradient, ldg, 0.0f, h, rows);
  if (rc) return rc;
  // 2. U = adam(H QR): the rotated gradient stays in the accumulators.
  {
    GemmProblem<float> prob = make_problem<float>(0, 0, m, n, n, h, rows, qr, ldqr, false);
    EpiAdam epi{momentum, variance, u, ldm, ldv, rows, sc};
    rc = launch_gemm<float>(s, prob, epi, 1);
    if (rc) return rc;
  }
  // 3. H = QL U
  rc = gemm<float>(s, 0, 0, m, n, m, 1.0f, ql, ldql, u, rows, 0.0f, h, rows);
  if (rc) return rc;
  // 4. update (row-major) = H QR^T, i.e. the column-major cols x rows matrix QR H^T.
  return gemm<float>(s, 0, 1, n, m, n, 1.0f, qr, ldqr, h, rows, 0.0f, update, ldu);
}

int soapmi_row_major_to_col_major_f32(const float* in, int64_t ldi, float* out, int64_t ldo, int64_t rows,
                                      int64_t cols, void* stream) {
  SOAPMI_REQUIRE(rows >= 0 && cols >= 0, "matrix dimensions must be non-negative");
  if (rows == 0 || cols == 0) return kOk;
  SOAPMI_REQUIRE(in && out, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(ldi >= cols && ldo >= rows, "leading dimensions are too small");
  // `in` is the column-major cols x rows matrix S; out = S^T.
  hipLaunchKernelGGL((transpose_kernel<float>), dim3((unsigned)ceil_div64(cols, 64), (unsigned)ceil_div64(rows, 64)),
                     dim3(256), 0, (hipStream_t)stream, in, ldi, out, ldo, (int)cols, (int)rows);
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

int soapmi_col_major_to_row_major_f32(const float* in, int64_t ldi, float* out, int64_t ldo, int64_t rows,
                                      int64_t cols, void* stream) {
  SOAPMI_REQUIRE(rows >= 0 && cols >= 0, "matrix dimensions must be non-negative");
  if (rows == 0 || cols == 0) return kOk;
  SOAPMI_REQUIRE(in && out, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(ldi >= rows && ldo >= cols, "leading dimensions are too small");
  hipLaunchKernelGGL((transpose_kernel<float>), dim3((unsigned)ceil_div64(rows, 64), (unsigned)ceil_div64(cols, 64)),
                     dim3(256), 0, (hipStream_t)stream, in, ldi, out, ldo, (int)rows, (int)cols);
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

}  // extern "C"
