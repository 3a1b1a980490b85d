// Stand-alone caller of the C ABI: no Python, no torch, only the HIP runtime for device memory.
//
//   abi_probe [rows cols [repeats [copies]]]
//   abi_probe qr n          QR of a pseudo-random n x n matrix (library-owned workspace), Q checked on the host
//   abi_probe eigh n        fp64 eigendecomposition of a symmetric n x n matrix, checked on the host
//   abi_probe eigh n [timed] two-stage   the eigh modes with the two-stage tridiagonalisation
//   abi_probe qr n [timed] two-level|three-level   the qr modes with the blocking fixed: 256-wide block reflectors
//                               only, or 1024-column super-blocks (left to the library: three levels up to n = 4096)
//   abi_probe burst             how the rate of one MFMA product (soapmi_gemm_f32, 11008 x 9984 x 1024, C -= A B) depends on what
//                               the device did just before: a steady stream of such products, the first ones after
//                               300 ms idle, and two of them alternating with 2.5 ms of idle, of tiny launches and
//                               of device-to-device copies (the pattern of a factorisation whose products sit
//                               between latency-bound panel phases)
//   abi_probe qr|eigh n timed   the same call four times, the last three timed, no host check (the
//                               check is cubic on one core: minutes at n = 11008)
//
// 1. `copies` layout copies of a rows x cols fp32 matrix (4*rows*cols bytes read, as many written):
//    the kernel of known size that hardware-counter readings of a profiled run are scaled by.
// 2. `repeats` calls of soapmi_rotate_adam_rotate_f32 (the update half of a steady-state step, four
//    MFMA products) with identity bases, so that the expected result is plain Adam on the gradient
//    and a sample of entries can be checked on the host in closed form.
// Prints the average time per call and the rate over the 4*rows*cols*(rows+cols) algorithmic flops;
// exits non-zero if any call fails or the sampled entries are off.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <unistd.h>
#include <string>
#include <vector>

#include "soap_mi355.h"

#define HIP_OK(expr)                                                                      \
  do {                                                                                    \
    hipError_t status_ = (expr);                                                          \
    if (status_ != hipSuccess) {                                                          \
      std::fprintf(stderr, "%s failed: %s\n", #expr, hipGetErrorString(status_));        \
      return 2;                                                                           \
    }                                                                                     \
  } while (0)

#define ABI_OK(expr)                                                                      \
  do {                                                                                    \
    int status_ = (expr);                                                                 \
    if (status_ != SOAPMI_OK) {                                                           \
      std::fprintf(stderr, "%s returned %d: %s\n", #expr, status_, soapmi_last_error()); \
      return 3;                                                                           \
    }                                                                                     \
  } while (0)

static float host_value(uint64_t index) {
  // cheap reproducible pseudo-random value in (-0.5, 0.5)
  uint64_t x = index * 0x9E3779B97F4A7C15ull + 0x632BE59BD9B4E019ull;
  x ^= x >> 29;
  x *= 0xBF58476D1CE4E5B9ull;
  x ^= x >> 32;
  return (float)((double)(x & 0xFFFFFF) / (double)0x1000000 - 0.5);
}

// Q^T Q = I and Q^T A upper triangular for soapmi_qr_f32 with a NULL workspace.  With timed_only the
// (cubic, single-threaded) host check is left out and the call is repeated between two events: the
// form a profiler run uses at large n.
static int check_qr(int64_t n, bool timed_only) {
  std::vector<float> a((size_t)n * n), q((size_t)n * n);
  for (size_t i = 0; i < a.size(); ++i) a[i] = host_value(i + 17);
  float *d_a, *d_q;
  HIP_OK(hipMalloc((void**)&d_a, a.size() * sizeof(float)));
  HIP_OK(hipMalloc((void**)&d_q, q.size() * sizeof(float)));
  HIP_OK(hipMemcpy(d_a, a.data(), a.size() * sizeof(float), hipMemcpyHostToDevice));
  ABI_OK(soapmi_qr_f32(d_a, d_q, n, n, n, nullptr, 0, nullptr));
  HIP_OK(hipDeviceSynchronize());
  if (timed_only) {
    hipEvent_t start, stop;
    HIP_OK(hipEventCreate(&start));
    HIP_OK(hipEventCreate(&stop));
    float total_ms = 0.0f;
    const int repeats = 3;
    for (int i = 0; i < repeats; ++i) {
      HIP_OK(hipMemcpy(d_a, a.data(), a.size() * sizeof(float), hipMemcpyHostToDevice));
      HIP_OK(hipEventRecord(start, nullptr));
      ABI_OK(soapmi_qr_f32(d_a, d_q, n, n, n, nullptr, 0, nullptr));
      HIP_OK(hipEventRecord(stop, nullptr));
      HIP_OK(hipEventSynchronize(stop));
      float ms = 0.0f;
      HIP_OK(hipEventElapsedTime(&ms, start, stop));
      total_ms += ms;
    }
    std::printf("qr n=%lld: %.3f ms per call (mean of %d)\n", (long long)n, total_ms / repeats, repeats);
    hipFree(d_a); hipFree(d_q);
    return 0;
  }
  HIP_OK(hipMemcpy(q.data(), d_q, q.size() * sizeof(float), hipMemcpyDeviceToHost));
  double worst_orth = 0.0, worst_lower = 0.0;
  for (int64_t i = 0; i < n; ++i)
    for (int64_t j = 0; j < n; ++j) {
      double dot = 0.0, r = 0.0;
      for (int64_t k = 0; k < n; ++k) {
        dot += (double)q[k + i * n] * q[k + j * n];
        r += (double)q[k + i * n] * a[k + j * n];  // R[i, j] = (Q^T A)[i, j]
      }
      worst_orth = std::fmax(worst_orth, std::fabs(dot - (i == j ? 1.0 : 0.0)));
      if (i > j) worst_lower = std::fmax(worst_lower, std::fabs(r));
    }
  std::printf("qr n=%lld: max |Q^T Q - I| %.3e, max |strictly lower (Q^T A)| %.3e\n", (long long)n, worst_orth,
              worst_lower);
  hipFree(d_a); hipFree(d_q);
  if (!(worst_orth < 1e-4 && worst_lower < 1e-4 * std::sqrt((double)n))) return 4;
  std::printf("ok\n");
  return 0;
}

// A Z = Z diag(w), Z^T Z = I, w ascending for soapmi_eigh_f64 with a NULL workspace.
static int check_eigh(int64_t n, bool timed_only) {
  std::vector<double> a((size_t)n * n), z((size_t)n * n), w((size_t)n);
  for (int64_t i = 0; i < n; ++i)
    for (int64_t j = 0; j <= i; ++j) a[i + j * n] = a[j + i * n] = host_value((uint64_t)(i * n + j) + 5);
  double *d_a, *d_z, *d_w;
  HIP_OK(hipMalloc((void**)&d_a, a.size() * sizeof(double)));
  HIP_OK(hipMalloc((void**)&d_z, z.size() * sizeof(double)));
  HIP_OK(hipMalloc((void**)&d_w, w.size() * sizeof(double)));
  HIP_OK(hipMemcpy(d_a, a.data(), a.size() * sizeof(double), hipMemcpyHostToDevice));
  ABI_OK(soapmi_eigh_f64(d_a, d_w, d_z, n, n, n, nullptr, 0, nullptr));
  HIP_OK(hipDeviceSynchronize());
  if (timed_only) {
    hipEvent_t start, stop;
    HIP_OK(hipEventCreate(&start));
    HIP_OK(hipEventCreate(&stop));
    float total_ms = 0.0f;
    const int repeats = 3;
    for (int i = 0; i < repeats; ++i) {
      HIP_OK(hipMemcpy(d_a, a.data(), a.size() * sizeof(double), hipMemcpyHostToDevice));
      HIP_OK(hipEventRecord(start, nullptr));
      ABI_OK(soapmi_eigh_f64(d_a, d_w, d_z, n, n, n, nullptr, 0, nullptr));
      HIP_OK(hipEventRecord(stop, nullptr));
      HIP_OK(hipEventSynchronize(stop));
      float ms = 0.0f;
      HIP_OK(hipEventElapsedTime(&ms, start, stop));
      total_ms += ms;
    }
    std::printf("eigh n=%lld: %.3f ms per call (mean of %d)\n", (long long)n, total_ms / repeats, repeats);
    hipFree(d_a); hipFree(d_z); hipFree(d_w);
    return 0;
  }
  HIP_OK(hipMemcpy(z.data(), d_z, z.size() * sizeof(double), hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(w.data(), d_w, w.size() * sizeof(double), hipMemcpyDeviceToHost));
  double worst_res = 0.0, worst_orth = 0.0, scale = 0.0;
  bool ascending = true;
  for (int64_t j = 0; j < n; ++j) {
    scale = std::fmax(scale, std::fabs(w[j]));
    if (j > 0 && w[j] < w[j - 1]) ascending = false;
  }
  for (int64_t j = 0; j < n; ++j) {
    for (int64_t i = 0; i < n; ++i) {
      double az = 0.0, dot = 0.0;
      for (int64_t k = 0; k < n; ++k) {
        az += a[i + k * n] * z[k + j * n];
        dot += z[k + i * n] * z[k + j * n];
      }
      worst_res = std::fmax(worst_res, std::fabs(az - w[j] * z[i + j * n]));
      worst_orth = std::fmax(worst_orth, std::fabs(dot - (i == j ? 1.0 : 0.0)));
    }
  }
  std::printf("eigh n=%lld: max |A Z - Z w| / max|w| %.3e, max |Z^T Z - I| %.3e, ascending %d\n", (long long)n,
              worst_res / scale, worst_orth, (int)ascending);
  hipFree(d_a); hipFree(d_z); hipFree(d_w);
  if (!(ascending && worst_res / scale < 1e-12 && worst_orth < 1e-12)) return 4;
  std::printf("ok\n");
  return 0;
}

// (The probe is built for the host only: it launches no kernels of its own.  Device buffers are filled from the
// host; the "tiny launch" is the library's layout copy of an 8 x 8 matrix.)
static int check_burst() {
  const int64_t M = 11008, N = 9984, K = 1024;
  float *a, *b, *c, *tiny;
  HIP_OK(hipMalloc((void**)&a, M * K * sizeof(float)));
  HIP_OK(hipMalloc((void**)&b, K * N * sizeof(float)));
  HIP_OK(hipMalloc((void**)&c, 2 * M * N * sizeof(float)));  // second half: target of the filler copies
  HIP_OK(hipMalloc((void**)&tiny, 512));
  HIP_OK(hipMemset(tiny, 0, 512));
  {
    std::vector<float> host((size_t)M * N);
    for (size_t i = 0; i < host.size(); ++i) host[i] = host_value(i);
    HIP_OK(hipMemcpy(c, host.data(), (size_t)M * N * sizeof(float), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(a, host.data(), (size_t)M * K * sizeof(float), hipMemcpyHostToDevice));
    for (size_t i = 0; i < (size_t)K * N; ++i) host[i] *= 1e-3f;
    HIP_OK(hipMemcpy(b, host.data(), (size_t)K * N * sizeof(float), hipMemcpyHostToDevice));
  }
  const double flops = 2.0 * (double)M * (double)N * (double)K;
  auto product = [&]() { return soapmi_gemm_f32(0, 0, M, N, K, -1.0f, a, M, b, K, 1.0f, c, M, nullptr); };
  hipEvent_t ev[64];
  for (auto& e : ev) HIP_OK(hipEventCreate(&e));
  auto report = [&](const char* what, double us) {
    std::printf("%-58s %7.0f us  %6.1f TFLOP/s\n", what, us, flops / us / 1e6);
  };
  // 1. after idle, then a steady stream
  for (int i = 0; i < 40; ++i) ABI_OK(product());
  HIP_OK(hipDeviceSynchronize());
  usleep(300000);
  for (int i = 0; i < 63; ++i) {
    HIP_OK(hipEventRecord(ev[i], nullptr));
    ABI_OK(product());
  }
  HIP_OK(hipEventRecord(ev[63], nullptr));
  HIP_OK(hipDeviceSynchronize());
  double first = 0.0, steady = 0.0;
  for (int i = 0; i < 63; ++i) {
    float ms = 0.0f;
    HIP_OK(hipEventElapsedTime(&ms, ev[i], ev[i + 1]));
    if (i < 3) first += ms * 1000.0 / 3.0;
    if (i >= 43) steady += ms * 1000.0 / 20.0;
  }
  report("first three products after 300 ms idle (mean)", first);
  report("products 44..63 of the same stream (mean)", steady);
  // 2. two products alternating with 2.5 ms of something else; the last of 14 rounds is reported
  const char* names[3] = {"two products after 2.5 ms idle, 14th round", "two products after 500 tiny launches, 14th round",
                          "two products after 12 device-to-device copies, 14th round"};
  for (int mode = 0; mode < 3; ++mode) {
    float ms = 0.0f;
    for (int round = 0; round < 14; ++round) {
      if (mode == 0) {
        HIP_OK(hipDeviceSynchronize());
        usleep(2500);
      } else if (mode == 1) {
        for (int i = 0; i < 500; ++i) ABI_OK(soapmi_row_major_to_col_major_f32(tiny, 8, tiny + 32, 8, 8, 8, nullptr));
      } else {
        for (int i = 0; i < 12; ++i)
          HIP_OK(hipMemcpyAsync(c + M * N, c + M * N / 2, (size_t)M * N * 2, hipMemcpyDeviceToDevice, nullptr));
      }
      HIP_OK(hipEventRecord(ev[0], nullptr));
      ABI_OK(product());
      ABI_OK(product());
      HIP_OK(hipEventRecord(ev[1], nullptr));
      HIP_OK(hipDeviceSynchronize());
      HIP_OK(hipEventElapsedTime(&ms, ev[0], ev[1]));
    }
    report(names[mode], ms * 500.0);
    for (int i = 0; i < 30; ++i) ABI_OK(product());  // back to the steady state before the next pattern
    HIP_OK(hipDeviceSynchronize());
  }
  hipFree(a); hipFree(b); hipFree(c); hipFree(tiny);
  std::printf("ok\n");
  return 0;
}

int main(int argc, char** argv) {
  if (argc == 2 && std::string(argv[1]) == "burst") return check_burst();
  // a trailing "two-stage" selects the two-stage tridiagonalisation for the eigh modes
  if (argc >= 4 && std::string(argv[1]) == "eigh" && std::string(argv[argc - 1]) == "two-stage") {
    ABI_OK(soapmi_set_option("eigh_algorithm", 2));
    --argc;
  }
  if (argc >= 4 && std::string(argv[1]) == "qr" &&
      (std::string(argv[argc - 1]) == "two-level" || std::string(argv[argc - 1]) == "three-level")) {
    ABI_OK(soapmi_set_option("qr_super_block", std::string(argv[argc - 1]) == "two-level" ? 256 : 1024));
    --argc;
  }
  const bool timed_only = argc == 4 && std::string(argv[3]) == "timed";
  if ((argc == 3 || timed_only) && std::string(argv[1]) == "qr") return check_qr(std::atoll(argv[2]), timed_only);
  if ((argc == 3 || timed_only) && std::string(argv[1]) == "eigh") return check_eigh(std::atoll(argv[2]), timed_only);
  const int64_t rows = argc > 2 ? std::atoll(argv[1]) : 4096;
  const int64_t cols = argc > 2 ? std::atoll(argv[2]) : 11008;
  const int repeats = argc > 3 ? std::atoi(argv[3]) : 5;
  const int copies = argc > 4 ? std::atoi(argv[4]) : 3;
  if (rows <= 0 || cols <= 0 || repeats <= 0 || copies < 0) {
    std::fprintf(stderr, "usage: abi_probe [rows cols [repeats [copies]]]  | abi_probe qr N [timed]  | abi_probe eigh N [timed]\n");
    return 1;
  }
  std::printf("backend %s, %lld x %lld, %d calls, %d calibration copies\n", soapmi_compiled_gpu_backend(),
              (long long)rows, (long long)cols, repeats, copies);
  std::fflush(stdout);

  const size_t mn = (size_t)rows * cols;
  std::vector<float> gradient(mn);
  for (size_t i = 0; i < mn; ++i) gradient[i] = host_value(i);
  std::vector<float> identity_l((size_t)rows * rows, 0.0f), identity_r((size_t)cols * cols, 0.0f);
  for (int64_t i = 0; i < rows; ++i) identity_l[(size_t)i * rows + i] = 1.0f;
  for (int64_t i = 0; i < cols; ++i) identity_r[(size_t)i * cols + i] = 1.0f;

  float *d_gradient, *d_update, *d_ql, *d_qr, *d_momentum, *d_variance, *d_copy;
  void* d_workspace;
  const size_t workspace_bytes = soapmi_rotate_adam_rotate_workspace_bytes(rows, cols);
  HIP_OK(hipMalloc((void**)&d_gradient, mn * sizeof(float)));
  HIP_OK(hipMalloc((void**)&d_update, mn * sizeof(float)));
  HIP_OK(hipMalloc((void**)&d_copy, mn * sizeof(float)));
  HIP_OK(hipMalloc((void**)&d_momentum, mn * sizeof(float)));
  HIP_OK(hipMalloc((void**)&d_variance, mn * sizeof(float)));
  HIP_OK(hipMalloc((void**)&d_ql, identity_l.size() * sizeof(float)));
  HIP_OK(hipMalloc((void**)&d_qr, identity_r.size() * sizeof(float)));
  HIP_OK(hipMalloc(&d_workspace, workspace_bytes));
  HIP_OK(hipMemcpy(d_gradient, gradient.data(), mn * sizeof(float), hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_ql, identity_l.data(), identity_l.size() * sizeof(float), hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_qr, identity_r.data(), identity_r.size() * sizeof(float), hipMemcpyHostToDevice));
  HIP_OK(hipMemset(d_momentum, 0, mn * sizeof(float)));
  HIP_OK(hipMemset(d_variance, 0, mn * sizeof(float)));

  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  for (int c = 0; c < copies; ++c)
    ABI_OK(soapmi_row_major_to_col_major_f32(d_gradient, cols, d_copy, rows, rows, cols, stream));

  const double beta1 = 0.95, beta2 = 0.95, eps = 1e-8;
  hipEvent_t begin, end;
  HIP_OK(hipEventCreate(&begin));
  HIP_OK(hipEventCreate(&end));
  // first call untimed (step 1), then `repeats` timed calls (steps 2 ..)
  ABI_OK(soapmi_rotate_adam_rotate_f32(d_gradient, cols, d_update, cols, d_ql, rows, d_qr, cols, d_momentum, rows,
                                       d_variance, rows, rows, cols, 1, beta1, beta2, eps, d_workspace,
                                       workspace_bytes, stream));
  HIP_OK(hipEventRecord(begin, stream));
  for (int r = 0; r < repeats; ++r)
    ABI_OK(soapmi_rotate_adam_rotate_f32(d_gradient, cols, d_update, cols, d_ql, rows, d_qr, cols, d_momentum, rows,
                                         d_variance, rows, rows, cols, 2 + r, beta1, beta2, eps, d_workspace,
                                         workspace_bytes, stream));
  HIP_OK(hipEventRecord(end, stream));
  HIP_OK(hipStreamSynchronize(stream));
  float elapsed_ms = 0.0f;
  HIP_OK(hipEventElapsedTime(&elapsed_ms, begin, end));
  const double per_call_ms = elapsed_ms / repeats;
  const double flops = 4.0 * (double)rows * (double)cols * (double)(rows + cols);
  std::printf("rotate_adam_rotate: %.3f ms per call, %.1f TFLOP/s over 4mn(m+n) flops\n", per_call_ms,
              flops / (per_call_ms * 1e-3) / 1e12);

  // With identity bases and a constant gradient g, after t steps m = (1-b1^t) g, v = (1-b2^t) g^2,
  // so the update is g / (|g| + eps / sqrt(1-b2^t)) for every entry.
  std::vector<float> update(mn);
  HIP_OK(hipMemcpy(update.data(), d_update, mn * sizeof(float), hipMemcpyDeviceToHost));
  const int steps = 1 + repeats;
  const double bc2 = 1.0 - std::pow(beta2, steps);
  double worst = 0.0;
  const size_t stride = mn / 4099 + 1;
  for (size_t i = 0; i < mn; i += stride) {
    const double g = gradient[i];
    const double expected = g / (std::fabs(g) + eps / std::sqrt(bc2));
    worst = std::fmax(worst, std::fabs((double)update[i] - expected));
  }
  std::printf("closed-form check on %zu sampled entries: max abs error %.3e\n", (mn + stride - 1) / stride, worst);
  if (!(worst < 2e-4)) {
    std::fprintf(stderr, "update differs from the closed form\n");
    return 4;
  }
  hipFree(d_gradient); hipFree(d_update); hipFree(d_copy); hipFree(d_momentum); hipFree(d_variance);
  hipFree(d_ql); hipFree(d_qr); hipFree(d_workspace);
  std::printf("ok\n");
  return 0;
}
