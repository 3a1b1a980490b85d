// Blocked Householder tridiagonalisation of a dense symmetric matrix (LAPACK sytrd/latrd scheme,
// lower storage), the first stage of the eigensolver that replaces ELPA's one-stage solver
// (src/soap_tp/csrc/elpa_bindings.cpp:149,165).
//
// Per column j of a panel four launches run, each ending where a matrix-wide reduction is needed:
//   A  finish the previous w (w += alpha2 v), bring column j up to date with the panel's pending
//      rank-2 updates, partial sums of the sub-column norm
//   B  reflector scalars (every workgroup re-derives them from the same partial sums), v, and
//      partial products W^T v, V^T v
//   C  y = A_trailing v : the bandwidth-bound kernel; a workgroup owns 256 rows x one column chunk,
//      lanes run along rows so every load instruction reads 512 contiguous bytes
//   D  w = tau (y - V (W^T v) - W (V^T v)) and partial sums of w^T v
// The trailing matrix keeps both triangles valid (the rank-2k update runs on the MFMA GEMM over
// the full square), so kernel C is a plain column-major matrix-vector product.
// All cross-workgroup reductions are "write partials, every consumer re-sums them in the same
// order": no atomics, reproducible results.
#pragma once
#include "common.hpp"
#include "gemm.hpp"
#include "qr.hpp"

namespace soapmi {

constexpr int kTrdNb = 32;        // panel width
constexpr int kTrdMaxChunks = 32; // column chunks of the matrix-vector product

template <typename T>
struct TrdWorkspace {
  T* vc;        // n x NB   clean reflector block of the current panel (rows are global indices)
  T* w;         // n x NB
  T* y_part;    // kTrdMaxChunks x n
  T* norm_part; // nwg
  T* dot_part;  // nwg
  T* t_part;    // nwg x 2*NB   partial (W^T v | V^T v)
  T* scal;      // small: [0] tau_j  [1] alpha2 (unused slots spare)
  int nwg;
};

template <typename T, class WS>
static inline void trd_workspace_layout(WS& ws, int64_t n, TrdWorkspace<T>* out) {
  const int64_t nwg = ceil_div64(n, 256);
  T* vc = ws.template take<T>((size_t)n * kTrdNb);
  T* w = ws.template take<T>((size_t)n * kTrdNb);
  T* y_part = ws.template take<T>((size_t)n * kTrdMaxChunks);
  T* norm_part = ws.template take<T>((size_t)nwg);
  T* dot_part = ws.template take<T>((size_t)nwg);
  T* t_part = ws.template take<T>((size_t)nwg * 2 * kTrdNb);
  T* scal = ws.template take<T>(16);
  if (out) *out = TrdWorkspace<T>{vc, w, y_part, norm_part, dot_part, t_part, scal, (int)nwg};
}

template <typename T>
__device__ __forceinline__ T block_sum_256(T v, T* red) {
  const int tid = threadIdx.x;
  red[tid] = v;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if (tid < s) red[tid] += red[tid + s];
    __syncthreads();
  }
  const T r = red[0];
  __syncthreads();
  return r;
}

// Sum of `count` per-workgroup partials, computed by the whole 256-thread workgroup in a fixed
// order (strided partial sums, then a tree), so every workgroup obtains the same bits.
template <typename T>
__device__ __forceinline__ T reduce_partials(const T* __restrict__ part, int count, T* red) {
  T s = T(0);
  for (int i = threadIdx.x; i < count; i += 256) s += part[i];
  return block_sum_256(s, red);
}

// Kernel A.  Rows r >= j.  i = j - p is the number of reflectors already in the panel.
//  - if i > 0: W[:, i-1] += alpha2 * Vc[:, i-1] with alpha2 = -tau_prev/2 * sum(dot_part)
//  - a_j[r] -= sum_{k<i} Vc[r,k] W[j,k] + W[r,k] Vc[j,k]
//  - d[j] = a_j[j]; partial norm over rows > j+1
template <typename T>
__global__ __launch_bounds__(256) void trd_col_update_kernel(T* __restrict__ A, int64_t lda, int n, int p, int j,
                                                             T* __restrict__ Vc, T* __restrict__ W, int64_t ldw,
                                                             const T* __restrict__ dot_part, int n_dot_part,
                                                             const T* __restrict__ tau, T* __restrict__ norm_part,
                                                             T* __restrict__ d) {
  constexpr int NB = kTrdNb;
  __shared__ T red[256];
  __shared__ T s_wj[NB], s_vj[NB];
  const int tid = threadIdx.x;
  const int i = j - p;
  const int r = j + blockIdx.x * 256 + tid;
  const bool live = r < n;
  T alpha2 = T(0);
  if (i > 0) alpha2 = T(-0.5) * tau[j - 1] * reduce_partials(dot_part, n_dot_part, red);
  // row j of W and Vc (finalising column i-1 of W on the fly)
  if (tid < i) {
    T wv = W[j + (int64_t)tid * ldw];
    const T vv = Vc[j + (int64_t)tid * ldw];
    if (tid == i - 1) wv += alpha2 * vv;
    s_wj[tid] = wv;
    s_vj[tid] = vv;
  }
  __syncthreads();
  T x2 = T(0);
  if (live) {
    // all 2*NB loads are issued before the first use (fixed trip count, guarded by k < i)
    T wr[NB], vr[NB];
#pragma unroll
    for (int k = 0; k < NB; ++k) {
      wr[k] = (k < i) ? W[r + (int64_t)k * ldw] : T(0);
      vr[k] = (k < i) ? Vc[r + (int64_t)k * ldw] : T(0);
    }
    T acc = T(0);
#pragma unroll
    for (int k = 0; k < NB; ++k) {
      if (k < i) {
        T wk = wr[k];
        if (k == i - 1) {
          wk += alpha2 * vr[k];
          // Row j stays unfinished in memory: every workgroup reads it above and adds alpha2
          // itself, and no later column looks at row j of W again.
          if (r != j) W[r + (int64_t)k * ldw] = wk;
        }
        acc += vr[k] * s_wj[k] + wk * s_vj[k];
      }
    }
    T a = A[r + (int64_t)j * lda];
    if (i > 0) {
      a -= acc;
      A[r + (int64_t)j * lda] = a;
    }
    if (r == j) d[j] = a;
    if (r > j + 1) x2 = a * a;
  }
  const T s = block_sum_256(x2, red);
  if (tid == 0) norm_part[blockIdx.x] = s;
}

// Rows of W below the current column that kernel A of this launch did not touch must also be
// finalised before the rank-2k update; this runs once per panel after its last column.
template <typename T>
__global__ __launch_bounds__(256) void trd_finish_w_kernel(T* __restrict__ W, const T* __restrict__ Vc, int64_t ldw,
                                                           int n, int row0, int col, const T* __restrict__ dot_part,
                                                           int n_dot_part, const T* __restrict__ tau_prev) {
  __shared__ T red[256];
  const int r = row0 + blockIdx.x * blockDim.x + threadIdx.x;
  const T alpha2 = T(-0.5) * tau_prev[0] * reduce_partials(dot_part, n_dot_part, red);
  if (r >= n) return;
  W[r + (int64_t)col * ldw] += alpha2 * Vc[r + (int64_t)col * ldw];
}

// Kernel B.  Rows r >= j+1 (workgroup/thread mapping: r = j + 1 + ...).
template <typename T>
__global__ __launch_bounds__(256) void trd_reflector_kernel(T* __restrict__ A, int64_t lda, int n, int p, int j,
                                                            T* __restrict__ Vc, const T* __restrict__ W, int64_t ldw,
                                                            const T* __restrict__ norm_part, int n_norm_part,
                                                            T* __restrict__ tau, T* __restrict__ e,
                                                            T* __restrict__ t_part) {
  constexpr int NB = kTrdNb;
  __shared__ T s_red[4][2 * NB];
  __shared__ T red[256];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int i = j - p;
  const int r = j + 1 + blockIdx.x * 256 + tid;
  const bool live = r < n;
  const T x2 = reduce_partials(norm_part, n_norm_part, red);
  const T alpha = A[(j + 1) + (int64_t)j * lda];
  T beta = alpha, tauv = T(0), scale = T(0);
  if (x2 > T(0)) {
    const T nrm = sqrt(alpha * alpha + x2);
    beta = (alpha >= T(0)) ? -nrm : nrm;
    tauv = (beta - alpha) / beta;
    scale = T(1) / (alpha - beta);
  }
  T v = T(0);
  if (live) {
    if (r == j + 1) {
      v = T(1);
    } else {
      v = A[r + (int64_t)j * lda] * scale;
    }
  }
  // everything that reads A[j+1, j] has done so before it is overwritten below
  __syncthreads();
  if (live) {
    if (r == j + 1) {
      tau[j] = tauv;
      e[j] = beta;
    } else {
      A[r + (int64_t)j * lda] = v;  // reflector kept for the back-transformation
    }
    Vc[r + (int64_t)i * ldw] = v;
  }
  // rows <= j of this column of Vc must read as zero for later row-j lookups
  if (blockIdx.x == 0) {
    for (int rr = p + tid; rr <= j; rr += 256) Vc[rr + (int64_t)i * ldw] = T(0);
  }
  // partial W^T v and V^T v over this workgroup's rows (columns k < i): 2*NB products per thread,
  // two 32-value butterflies per wavefront
  {
    T pw[NB], pv[NB];
#pragma unroll
    for (int k = 0; k < NB; ++k) {
      const bool on = live && k < i;
      pw[k] = on ? W[r + (int64_t)k * ldw] * v : T(0);
      pv[k] = on ? Vc[r + (int64_t)k * ldw] * v : T(0);
    }
    const T tw = wave_reduce_32<T>(pw, lane);
    const T tv = wave_reduce_32<T>(pv, lane);
    if ((lane & 1) == 0) {
      s_red[wave][(lane >> 1) & 31] = tw;
      s_red[wave][NB + ((lane >> 1) & 31)] = tv;
    }
  }
  __syncthreads();
  if (tid < 2 * NB) {
    const int k = tid % NB;
    T s = T(0);
    if (k < i) s = s_red[0][tid] + s_red[1][tid] + s_red[2][tid] + s_red[3][tid];
    t_part[(int64_t)blockIdx.x * 2 * NB + tid] = s;
  }
}

// Kernel C.  y_part[chunk][r] = sum over this chunk's columns of A[r, c] v[c];  rows and columns
// both run over j+1 .. n-1.  v is read from column i of Vc.
template <typename T>
__global__ __launch_bounds__(256) void trd_symv_kernel(const T* __restrict__ A, int64_t lda, int n, int j,
                                                       const T* __restrict__ v, T* __restrict__ y_part, int chunk_w) {
  __shared__ T s_v[512];
  const int tid = threadIdx.x;
  const int r = j + 1 + blockIdx.x * 256 + tid;
  const int c_begin = j + 1 + blockIdx.y * chunk_w;
  const int c_end = min(n, c_begin + chunk_w);
  T acc0 = T(0), acc1 = T(0), acc2 = T(0), acc3 = T(0);
  for (int cb = c_begin; cb < c_end; cb += 512) {
    const int cnt = min(512, c_end - cb);
    __syncthreads();
    for (int t = tid; t < cnt; t += 256) s_v[t] = v[cb + t];
    __syncthreads();
    if (r < n) {
      const T* col = A + r + (int64_t)cb * lda;
      int c = 0;
      for (; c + 4 <= cnt; c += 4) {
        const T a0 = col[(int64_t)(c + 0) * lda];
        const T a1 = col[(int64_t)(c + 1) * lda];
        const T a2 = col[(int64_t)(c + 2) * lda];
        const T a3 = col[(int64_t)(c + 3) * lda];
        acc0 += a0 * s_v[c + 0];
        acc1 += a1 * s_v[c + 1];
        acc2 += a2 * s_v[c + 2];
        acc3 += a3 * s_v[c + 3];
      }
      for (; c < cnt; ++c) acc0 += col[(int64_t)c * lda] * s_v[c];
    }
  }
  if (r < n) y_part[(int64_t)blockIdx.y * n + r] = (acc0 + acc1) + (acc2 + acc3);
}

// Kernel D.  Rows r >= j+1.
template <typename T>
__global__ __launch_bounds__(256) void trd_w_kernel(int n, int p, int j, const T* __restrict__ Vc, T* __restrict__ W,
                                                    int64_t ldw, const T* __restrict__ y_part, int n_chunks,
                                                    const T* __restrict__ t_part, int n_t_part,
                                                    const T* __restrict__ tau, T* __restrict__ dot_part) {
  constexpr int NB = kTrdNb;
  __shared__ T red[256];
  __shared__ T s_t[2 * NB];
  __shared__ T s_t4[4][2 * NB];
  const int tid = threadIdx.x;
  const int i = j - p;
  const int r = j + 1 + blockIdx.x * 256 + tid;
  {
    // 2*NB columns x n_t_part partials: 4 strided partial sums per column, then 4 adds
    const int c = tid & (2 * NB - 1), g0 = tid >> 6;
    T s = T(0);
    if ((c % NB) < i)
      for (int g = g0; g < n_t_part; g += 4) s += t_part[(int64_t)g * 2 * NB + c];
    s_t4[g0][c] = s;
  }
  __syncthreads();
  if (tid < 2 * NB) s_t[tid] = (s_t4[0][tid] + s_t4[1][tid]) + (s_t4[2][tid] + s_t4[3][tid]);
  __syncthreads();
  T prod = T(0);
  if (r < n) {
    T yp[kTrdMaxChunks], wr[NB], vr[NB];
#pragma unroll
    for (int c = 0; c < kTrdMaxChunks; ++c) yp[c] = (c < n_chunks) ? y_part[(int64_t)c * n + r] : T(0);
#pragma unroll
    for (int k = 0; k < NB; ++k) {
      vr[k] = (k < i) ? Vc[r + (int64_t)k * ldw] : T(0);
      wr[k] = (k < i) ? W[r + (int64_t)k * ldw] : T(0);
    }
    T y = T(0);
#pragma unroll
    for (int c = 0; c < kTrdMaxChunks; ++c) y += yp[c];
    T corr = T(0);
#pragma unroll
    for (int k = 0; k < NB; ++k) corr += vr[k] * s_t[k] + wr[k] * s_t[NB + k];
    const T wv = tau[j] * (y - corr);
    W[r + (int64_t)i * ldw] = wv;
    prod = wv * Vc[r + (int64_t)i * ldw];
  }
  const T s = block_sum_256(prod, red);
  if (tid == 0) dot_part[blockIdx.x] = s;
}

// d[n-1] after all updates: the last column has no reflector of its own.
// Tridiagonalise A (n x n, both triangles valid on entry; destroyed).  On exit d[0..n), e[0..n-1),
// tau[0..n-1) and, below the first subdiagonal of A, the reflector vectors (implicit unit at
// row j+1 of column j), as LAPACK sytrd('L') leaves them.
template <typename T>
static inline int sytrd_lower(hipStream_t s, T* A, int64_t lda, int n, T* d, T* e, T* tau, const TrdWorkspace<T>& ws) {
  constexpr int NB = kTrdNb;
  const int64_t ldw = n;
  if (n == 1) {
    SOAPMI_HIP(hipMemcpyAsync(d, A, sizeof(T), hipMemcpyDeviceToDevice, s));
    return kOk;
  }
  int last_dot_parts = 0;  // number of dot partials produced by the latest kernel D
  for (int p = 0; p < n; p += NB) {
    const int pe = std::min(n, p + NB);
    int cols_done = 0;
    for (int j = p; j < pe; ++j) {
      const int i = j - p;
      const int nwgA = (int)ceil_div64(n - j, 256);
      hipLaunchKernelGGL((trd_col_update_kernel<T>), dim3(nwgA), dim3(256), 0, s, A, lda, n, p, j, ws.vc, ws.w, ldw,
                         ws.dot_part, last_dot_parts, tau, ws.norm_part, d);
      if (j == n - 1) break;  // only the diagonal entry remained
      const int nt = n - j - 1;
      const int nwgB = (int)ceil_div64(nt, 256);
      hipLaunchKernelGGL((trd_reflector_kernel<T>), dim3(nwgB), dim3(256), 0, s, A, lda, n, p, j, ws.vc, ws.w, ldw,
                         ws.norm_part, nwgA, tau, e, ws.t_part);
      int chunks = (int)std::min<int64_t>(kTrdMaxChunks, ceil_div64(nt, 64));
      const int chunk_w = (int)ceil_div64(nt, chunks);
      chunks = (int)ceil_div64(nt, chunk_w);
      hipLaunchKernelGGL((trd_symv_kernel<T>), dim3(nwgB, chunks), dim3(256), 0, s, A, lda, n, j,
                         ws.vc + (int64_t)i * ldw, ws.y_part, chunk_w);
      hipLaunchKernelGGL((trd_w_kernel<T>), dim3(nwgB), dim3(256), 0, s, n, p, j, ws.vc, ws.w, ldw, ws.y_part, chunks,
                         ws.t_part, nwgB, tau, ws.dot_part);
      last_dot_parts = nwgB;
      cols_done = i + 1;
    }
    SOAPMI_LAUNCH_CHECK();
    if (pe >= n) break;
    // finish the last w of the panel, then A[pe:, pe:] -= V W^T + W V^T on the full square
    const int jl = pe - 1;
    hipLaunchKernelGGL((trd_finish_w_kernel<T>), dim3((unsigned)ceil_div64(n - pe, 256)), dim3(256), 0, s, ws.w, ws.vc,
                       ldw, n, pe, cols_done - 1, ws.dot_part, last_dot_parts, tau + jl);
    last_dot_parts = 0;
    const int nt = n - pe;
    int rc = gemm<T>(s, 0, 1, nt, nt, cols_done, T(-1), ws.vc + pe, ldw, ws.w + pe, ldw, T(1),
                     A + pe + (int64_t)pe * lda, lda);
    if (rc) return rc;
    rc = gemm<T>(s, 0, 1, nt, nt, cols_done, T(-1), ws.w + pe, ldw, ws.vc + pe, ldw, T(1), A + pe + (int64_t)pe * lda,
                 lda);
    if (rc) return rc;
  }
  return kOk;
}

}  // namespace soapmi
