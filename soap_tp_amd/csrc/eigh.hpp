// Dense symmetric eigensolver: tridiagonalise (sytrd.hpp), divide and conquer on the tridiagonal
// matrix (stedc.hpp), back-transform the eigenvectors with the stored reflectors (compact-WY
// blocks on the MFMA GEMM).  Same three stages as the one-stage ELPA solver the reference calls
// (src/soap_tp/csrc/elpa_bindings.cpp:149,165); eigenvalues come back ascending.
#pragma once
#include "common.hpp"
#include "gemm.hpp"
#include "qr.hpp"
#include "stedc.hpp"
#include "sytrd.hpp"
#include "twostage.hpp"

namespace soapmi {

// Which tridiagonalisation the eigensolver uses.
enum : int { kEighOneStage = 1, kEighTwoStage = 2 };

template <typename T>
struct EighWorkspace {
  T* d;
  T* e;
  T* tau;
  TrdWorkspace<T> trd;
  DcWorkspace<T> dc;
  BlockReflectorWs<T> br;  // block-reflector scratch for the back-transformation
  T* t_block;              // kBrMax x kBrMax
  TwoStageWorkspace<T> ts; // only laid out for the two-stage algorithm
};

template <typename T, class WS>
static inline void eigh_workspace_layout(WS& ws, int64_t n, EighWorkspace<T>* out, int algorithm = kEighOneStage) {
  EighWorkspace<T> w;
  w.d = ws.template take<T>(n);
  w.e = ws.template take<T>(n);
  w.tau = ws.template take<T>(n);
  trd_workspace_layout<T>(ws, n, out ? &w.trd : nullptr);
  dc_workspace_layout<T>(ws, n, out ? &w.dc : nullptr);
  block_reflector_layout<T>(ws, n, out ? &w.br : nullptr);
  w.t_block = ws.template take<T>(kBrMax * kBrMax);
  if (algorithm == kEighTwoStage) two_stage_workspace_layout<T>(ws, n, out ? &w.ts : nullptr);
  if (out) *out = w;
}

template <typename T>
static inline size_t eigh_workspace_bytes(int64_t n, int algorithm = kEighOneStage) {
  WorkspaceSizer sizer;
  eigh_workspace_layout<T>(sizer, n, nullptr, algorithm);
  return sizer.total();
}

// w[0..n) and the diagonal of Z <- NaN if the tridiagonalisation reported lost messages: the
// decomposition is then unusable, and this makes it impossible to miss.  The host-visible report
// word (pinned host memory, may be null) is raised as well.
template <typename T>
__global__ void eigh_poison_on_error_kernel(T* __restrict__ w, T* __restrict__ Z, int64_t ldz, int n,
                                            const int* __restrict__ error, int* __restrict__ report) {
  if (*error == 0) return;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (report && i == 0) *report = 1;
  if (i < n) {
    w[i] = T(NAN);
    Z[i + (int64_t)i * ldz] = T(NAN);
  }
}

// out[i, j] = (Tout) in[i, reverse ? n-1-j : j]
template <typename Tin, typename Tout>
__global__ void convert_columns_kernel(const Tin* __restrict__ in, int64_t ldi, Tout* __restrict__ out, int64_t ldo,
                                       int n, int reverse) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  for (int j = blockIdx.y; j < n; j += gridDim.y) {
    const int sj = reverse ? n - 1 - j : j;
    out[i + (int64_t)j * ldo] = (Tout)in[i + (int64_t)sj * ldi];
  }
}

// The two-stage variant of eigh_ascending: dense -> band -> tridiagonal, divide and conquer, two
// back-transformations (twostage.hpp).  No persistent kernels: nothing here waits inside a kernel.
template <typename T>
static inline int eigh_ascending_two_stage(hipStream_t s, T* A, int64_t lda, T* w, T* Z, int64_t ldz, int n,
                                           const EighWorkspace<T>& ws) {
  const TwoStageWorkspace<T>& ts = ws.ts;
  int rc = sy2sb_lower<T>(s, A, lda, n, ts, ws.br, ws.t_block);
  if (rc) return rc;
  hipLaunchKernelGGL((sb_pack_band_kernel<T>), dim3((unsigned)ceil_div64(n, 4)), dim3(256), 0, s, A, lda, n, ts.ab);
  SOAPMI_LAUNCH_CHECK();
  rc = sb2st<T>(s, n, ts, ws.d, ws.e);
  if (rc) return rc;
  hipLaunchKernelGGL((fill_zero_wide_kernel<T>), dim3(4096), dim3(256), 0, s, ts.zpad, ts.ldz * (int64_t)n);
  SOAPMI_LAUNCH_CHECK();
  rc = stedc<T>(s, n, ws.d, ws.e, w, ts.zpad, ts.ldz, ws.dc);
  if (rc) return rc;
  rc = sb_apply_q2<T>(s, n, ts);
  if (rc) return rc;
  rc = sb_apply_q1<T>(s, A, lda, n, ts, ws.br, ws.t_block);
  if (rc) return rc;
  hipLaunchKernelGGL((convert_columns_kernel<T, T>), dim3((unsigned)ceil_div64(n, 256), (unsigned)(n < 4096 ? n : 4096)),
                     dim3(256), 0, s, ts.zpad, ts.ldz, Z, ldz, n, 0);
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

// A (n x n, lower triangle referenced, destroyed) = Z diag(w) Z^T, w ascending.
template <typename T>
static inline int eigh_ascending(hipStream_t s, T* A, int64_t lda, T* w, T* Z, int64_t ldz, int n,
                                 const EighWorkspace<T>& ws, unsigned spin_limit = kQrSpinLimit,
                                 int* report = nullptr, int algorithm = kEighOneStage) {
  if (n <= 0) return kOk;
  if (algorithm == kEighTwoStage && n >= 3) return eigh_ascending_two_stage<T>(s, A, lda, w, Z, ldz, n, ws);
  int rc = sytrd_lower<T>(s, A, lda, n, ws.d, ws.e, ws.tau, ws.trd, spin_limit);
  if (rc) return rc;
  rc = stedc<T>(s, n, ws.d, ws.e, w, Z, ldz, ws.dc);
  if (rc) return rc;
  // Z <- H_0 H_1 ... H_{n-2} Z, kBrMax-wide block reflectors applied last block first.
  const int nref = n - 1;  // reflector j lives in column j, rows j+1..n-1
  if (nref <= 0) return kOk;  // n == 1: no column kernel ran
  constexpr int OB = kBrMax;
  const int blocks = (int)ceil_div64(nref, OB);
  const int64_t ldv = n;
  for (int bi = blocks - 1; bi >= 0; --bi) {
    const int p = bi * OB, pe = std::min(nref, p + OB), nbw = pe - p;
    // The block's reflectors start in row p + 1; row p (all zero in V) is carried along so that the
    // products' row extent n - p stays a multiple of the MFMA tile whenever n and the block width are
    // (the fast product path), instead of one short of it.
    const int rows = n - p;
    launch_extract_v<T>(s, A, lda, rows, p, p, nbw, ws.br.v, ldv, 1);
    SOAPMI_LAUNCH_CHECK();
    rc = build_t_factor<T>(s, ws.br, rows, nbw, ldv, ws.tau + p, ws.t_block);
    if (rc) return rc;
    rc = apply_block_reflector<T>(s, ws.br, ws.t_block, false, rows, nbw, n, ldv, Z + p, ldz);
    if (rc) return rc;
  }
  hipLaunchKernelGGL((eigh_poison_on_error_kernel<T>), dim3((unsigned)ceil_div64(n, 256)), dim3(256), 0, s, w, Z, ldz, n,
                     ws.trd.error, report);
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

// out[i, j] = scale * (T_out) in[max(i,j), min(i,j)] (+ shift on the diagonal): builds the full
// symmetric solver input from the lower triangle of P, converting precision on the way.  One
// workgroup per 64 x 64 tile on or below the diagonal (grid: tiles x tiles, the others return at
// once): the tile is read with lanes along rows, written as it is and, transposed through LDS,
// onto its mirror image, so that every access to either matrix is coalesced.
template <typename Tin, typename Tout>
__global__ __launch_bounds__(256) void sym_convert_kernel(const Tin* __restrict__ in, int64_t ldi, Tout* __restrict__ out,
                                                          int64_t ldo, int n, Tout scale, Tout diag_shift) {
  __shared__ Tout tile[64][65];
  const int bi = blockIdx.x, bj = blockIdx.y;
  if (bi < bj) return;
  const int r0 = bi * 64, c0 = bj * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int c = ty; c < 64; c += 4) {
    const int gr = r0 + tx, gc = c0 + c;
    if (gr < n && gc < n) {
      const int r = gr > gc ? gr : gc, q = gr > gc ? gc : gr;  // only diagonal tiles hold entries above the diagonal
      Tout v = scale * (Tout)in[r + (int64_t)q * ldi];
      if (gr == gc) v += diag_shift;
      tile[c][tx] = v;
      out[gr + (int64_t)gc * ldo] = v;
    }
  }
  if (bi == bj) return;
  __syncthreads();
  for (int r = ty; r < 64; r += 4) {
    const int gr = r0 + r, gc = c0 + tx;
    if (gr < n && gc < n) out[gc + (int64_t)gr * ldo] = tile[tx][r];
  }
}

template <typename Tin, typename Tout>
__global__ void convert_vector_kernel(const Tin* __restrict__ in, Tout* __restrict__ out, int n, Tout scale,
                                      int reverse) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  out[i] = scale * (Tout)in[reverse ? n - 1 - i : i];
}

}  // namespace soapmi
