// Shared declarations for the gfx950 SOAP kernels: error plumbing, launch helpers,
// MFMA instruction traits.  Everything here targets CDNA4 (64-wide wavefronts) only.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

namespace soapmi {

// ---- status codes shared with include/soap_mi355.h ---------------------------------------
enum : int {
  kOk = 0,
  kInvalidArgument = -1,  // maps to ValueError on the Python side
  kRuntimeError = -2,     // maps to RuntimeError
  kNotConverged = -3,
  kWorkspaceTooSmall = -4,
};

void set_error(const char* fmt, ...);
const char* last_error();

#define SOAPMI_REQUIRE(cond, ...)            \
  do {                                       \
    if (!(cond)) {                           \
      ::soapmi::set_error(__VA_ARGS__);      \
      return ::soapmi::kInvalidArgument;     \
    }                                        \
  } while (0)

#define SOAPMI_HIP(call)                                                          \
  do {                                                                            \
    hipError_t e_ = (call);                                                       \
    if (e_ != hipSuccess) {                                                       \
      ::soapmi::set_error("%s failed: %s", #call, hipGetErrorString(e_));         \
      return ::soapmi::kRuntimeError;                                             \
    }                                                                             \
  } while (0)

#define SOAPMI_LAUNCH_CHECK()                                                     \
  do {                                                                            \
    hipError_t e_ = hipGetLastError();                                            \
    if (e_ != hipSuccess) {                                                       \
      ::soapmi::set_error("kernel launch failed: %s", hipGetErrorString(e_));     \
      return ::soapmi::kRuntimeError;                                             \
    }                                                                             \
  } while (0)

static inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Bump allocator over a caller-provided workspace.  Every sub-buffer is 256-byte aligned.
struct Workspace {
  char* base;
  size_t size;
  size_t used;
  Workspace(void* p, size_t n) : base(static_cast<char*>(p)), size(n), used(0) {}
  template <typename T>
  T* take(size_t count) {
    size_t off = align_up(used, 256);
    size_t bytes = count * sizeof(T);
    used = off + bytes;
    if (base == nullptr || used > size) return nullptr;
    return reinterpret_cast<T*>(base + off);
  }
};
// Size accounting twin of Workspace (used by the *_workspace_bytes queries).
struct WorkspaceSizer {
  size_t used = 0;
  template <typename T>
  T* take(size_t count) {
    used = align_up(used, 256) + count * sizeof(T);
    return nullptr;
  }
  size_t total() const { return align_up(used, 256) + 256; }
};

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef double f64x4 __attribute__((ext_vector_type(4)));

// MFMA traits.  Operand "a" is indexed by (row = lane % MI, k = lane / MI), operand "b" by
// (k = lane / MI, col = lane % MI).  Accumulator register r of lane l holds
// D[acc_row(r, l)][l % MI].  Both layouts were verified on gfx950 hardware against a host
// matrix product.
template <typename T>
struct Mfma;

template <>
struct Mfma<float> {
  static constexpr int MI = 32;    // tile edge
  static constexpr int KI = 2;     // k extent of one instruction
  static constexpr int NACC = 16;  // accumulator values per lane
  using Acc = f32x16;
  static __device__ __forceinline__ Acc mma(float a, float b, Acc c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ int acc_row(int r, int lane) {
    return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
  }
};

template <>
struct Mfma<double> {
  static constexpr int MI = 16;
  static constexpr int KI = 4;
  static constexpr int NACC = 4;
  using Acc = f64x4;
  static __device__ __forceinline__ Acc mma(double a, double b, Acc c) {
    return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ int acc_row(int r, int lane) { return (lane >> 4) + 4 * r; }
};

// 16-byte vector types used for global <-> LDS traffic.
template <typename T>
struct Vec16;
template <>
struct Vec16<float> {
  using type = float4;
  static constexpr int W = 4;
};
template <>
struct Vec16<double> {
  using type = double2;
  static constexpr int W = 2;
};

}  // namespace soapmi
