// Blocked Householder tridiagonalisation of a dense symmetric matrix (LAPACK sytrd/latrd scheme,
// lower storage), the first stage of the eigensolver that replaces ELPA's one-stage solver
// (src/soap_tp/csrc/elpa_bindings.cpp:149,165).
//
// Per column j of a panel four launches run, each ending where a matrix-wide reduction is needed:
//   A  finish the previous w (w += alpha2 v), bring column j up to date with the panel's pending
//      rank-2 updates, partial sums of the sub-column norm
//   B  reflector scalars (every workgroup re-derives them from the same partial sums), v, and
//      partial products W^T v, V^T v
//   C  y = A_trailing v : the bandwidth-bound kernel.  Only the lower triangle is read: a workgroup
//      owns one 128 x 128 tile on or below the diagonal and produces both the tile's product with
//      v (for its rows) and the transposed tile's product (for its columns, a wavefront butterfly
//      per 32 columns); lanes run along rows so every load instruction reads 512 contiguous bytes
//   D  w = tau (y - V (W^T v) - W (V^T v)) and partial sums of w^T v
// The rank-2k update of the trailing matrix runs on the MFMA product over the tiles on or below
// the diagonal only, as one product with K = 64: A -= [V | W] [W | V]^T.
// All cross-workgroup reductions are "write partials, every consumer re-sums them in the same
// order": no atomics, reproducible results.
#pragma once
#include "common.hpp"
#include "gemm.hpp"
#include "qr.hpp"

namespace soapmi {

constexpr int kTrdNb = 32;        // panel width
constexpr int kTrdTile = 128;     // tile edge of the matrix-vector product

template <typename T>
struct TrdWorkspace {
  T* vc;        // n x NB   clean reflector block of the current panel (rows are global indices)
  T* w;         // n x NB   directly behind vc: [vc | w] is one n x 2NB operand
  T* vc2;       // n x NB   copy of vc directly behind w: [w | vc2] is the other operand
  T* y_part;    // ceil(n / kTrdTile) x n   one slot per tile that touches an index
  T* norm_part; // nwg
  T* dot_part;  // nwg
  T* t_part;    // nwg x 2*NB   partial (W^T v | V^T v)
  T* scal;      // small: [0] tau_j  [1] alpha2 (unused slots spare)
  int nwg;
};

template <typename T, class WS>
static inline void trd_workspace_layout(WS& ws, int64_t n, TrdWorkspace<T>* out) {
  const int64_t nwg = ceil_div64(n, 256);
  // one allocation, so that the three blocks are adjacent whatever the allocator's alignment is
  T* vc = ws.template take<T>((size_t)3 * n * kTrdNb);
  T* w = vc + (size_t)n * kTrdNb;
  T* vc2 = w + (size_t)n * kTrdNb;
  T* y_part = ws.template take<T>((size_t)n * ceil_div64(n, kTrdTile));
  T* norm_part = ws.template take<T>((size_t)nwg);
  T* dot_part = ws.template take<T>((size_t)nwg);
  T* t_part = ws.template take<T>((size_t)nwg * 2 * kTrdNb);
  T* scal = ws.template take<T>(16);
  if (out) *out = TrdWorkspace<T>{vc, w, vc2, y_part, norm_part, dot_part, t_part, scal, (int)nwg};
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
                                                            T* __restrict__ Vc, T* __restrict__ Vc2,
                                                            const T* __restrict__ W, int64_t ldw,
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
    Vc2[r + (int64_t)i * ldw] = v;
  }
  // rows <= j of this column of Vc must read as zero for later row-j lookups
  if (blockIdx.x == 0) {
    for (int rr = p + tid; rr <= j; rr += 256) {
      Vc[rr + (int64_t)i * ldw] = T(0);
      Vc2[rr + (int64_t)i * ldw] = T(0);
    }
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

// Kernel C.  The trailing matrix (rows and columns o = j+1 .. n-1, only its lower triangle is
// valid) is cut into 128 x 128 tiles from its own origin; workgroup t owns tile (rb, cb), cb <= rb.
// 256 threads: thread (row = tid % 128, half = tid / 128) holds 64 entries of its row.  It adds
// a[row, c] v[c] to the row's sum ("direct") and, for the mirrored upper triangle, contributes
// a[row, c] v[row] to column c's sum, reduced over the rows by wavefront butterflies.
// y_part has one slot per tile edge: index i of block b receives slot s < b from tile (b, s)'s direct
// sums, slot s > b from tile (s, b)'s column sums, and slot b from the diagonal tile, which adds
// both.  Every (slot, index) pair is written exactly once, so kernel D sums nb slots per index in a
// fixed order and nothing has to be cleared.
template <typename T>
__global__ __launch_bounds__(256) void trd_symv_kernel(const T* __restrict__ A, int64_t lda, int n, int j,
                                                       const T* __restrict__ v, T* __restrict__ y_part) {
  constexpr int TS = kTrdTile;
  __shared__ T s_v[TS];
  __shared__ T s_direct[2][TS];
  __shared__ T s_col[4][64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // `half` is the same for all lanes of a wavefront: telling the compiler so moves the column
  // address arithmetic to the scalar unit
  const int row = tid & (TS - 1), half = __builtin_amdgcn_readfirstlane(tid >> 7);
  const int o = j + 1;
  const int t = blockIdx.x;
  int rb = (int)((sqrtf(8.0f * (float)t + 1.0f) - 1.0f) * 0.5f);
  while (rb * (rb + 1) / 2 > t) --rb;
  while ((rb + 1) * (rb + 2) / 2 <= t) ++rb;
  const int cb = t - rb * (rb + 1) / 2;
  const int r = o + rb * TS + row;        // global row of this thread
  const int c0 = o + cb * TS;             // first global column of the tile
  const bool live = r < n;
  const bool diagonal = rb == cb;
  if (tid < TS) s_v[tid] = (c0 + tid < n) ? v[c0 + tid] : T(0);
  const T vr = live ? v[r] : T(0);
  __syncthreads();
  T acc0 = T(0), acc1 = T(0);
  // Loads are unconditional on clamped addresses (always inside the matrix); what must not count
  // - rows past the end, the upper triangle inside a diagonal tile - is zeroed after the load.
  const int rr = min(r, n - 1);
  const int limit = diagonal ? r : n - 1;  // last column that counts for this row
#pragma unroll 1
  for (int q = 0; q < 2; ++q) {  // 32 columns at a time
    const int cq = c0 + 64 * half + 32 * q;
    T a[32];
#pragma unroll
    for (int k = 0; k < 32; ++k) a[k] = A[rr + (int64_t)min(cq + k, n - 1) * lda];
    T cols[32];
#pragma unroll
    for (int k = 0; k < 32; ++k) {
      const T x = (live && cq + k <= limit) ? a[k] : T(0);
      if (k & 1) acc1 += x * s_v[64 * half + 32 * q + k];
      else acc0 += x * s_v[64 * half + 32 * q + k];
      cols[k] = (diagonal && cq + k == r) ? T(0) : x * vr;  // the diagonal entry counts once
    }
    const T total = wave_reduce_32<T>(cols, lane);
    if ((lane & 1) == 0) s_col[wave][32 * q + ((lane >> 1) & 31)] = total;
  }
  s_direct[half][row] = acc0 + acc1;
  __syncthreads();
  if (tid < TS) {
    // wavefronts 2*half and 2*half+1 hold the two row halves of column half `half`
    const int h = tid >> 6, k = tid & 63;
    const T column_sum = s_col[2 * h][k] + s_col[2 * h + 1][k];
    const T row_sum = s_direct[0][tid] + s_direct[1][tid];
    const int gr = o + rb * TS + tid, gc = c0 + tid;
    if (diagonal) {
      if (gr < n) y_part[(int64_t)rb * n + gr] = row_sum + column_sum;
    } else {
      if (gr < n) y_part[(int64_t)cb * n + gr] = row_sum;
      if (gc < n) y_part[(int64_t)rb * n + gc] = column_sum;
    }
  }
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
    T wr[NB], vr[NB];
#pragma unroll
    for (int k = 0; k < NB; ++k) {
      vr[k] = (k < i) ? Vc[r + (int64_t)k * ldw] : T(0);
      wr[k] = (k < i) ? W[r + (int64_t)k * ldw] : T(0);
    }
    T y = T(0);
    for (int c0 = 0; c0 < n_chunks; c0 += 16) {  // 16 slot loads in flight, summed in slot order
      T yp[16];
#pragma unroll
      for (int c = 0; c < 16; ++c) yp[c] = (c0 + c < n_chunks) ? y_part[(int64_t)(c0 + c) * n + r] : T(0);
#pragma unroll
      for (int c = 0; c < 16; ++c) y += yp[c];
    }
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
// Tridiagonalise A (n x n, lower triangle referenced; destroyed).  On exit d[0..n), e[0..n-1),
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
      hipLaunchKernelGGL((trd_reflector_kernel<T>), dim3(nwgB), dim3(256), 0, s, A, lda, n, p, j, ws.vc, ws.vc2, ws.w,
                         ldw, ws.norm_part, nwgA, tau, e, ws.t_part);
      const int nb = (int)ceil_div64(nt, kTrdTile);
      hipLaunchKernelGGL((trd_symv_kernel<T>), dim3(nb * (nb + 1) / 2), dim3(256), 0, s, A, lda, n, j,
                         ws.vc + (int64_t)i * ldw, ws.y_part);
      hipLaunchKernelGGL((trd_w_kernel<T>), dim3(nwgB), dim3(256), 0, s, n, p, j, ws.vc, ws.w, ldw, ws.y_part, nb,
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
    // A[pe:, pe:] -= [V | W] [W | V]^T, tiles on or below the diagonal only
    int rc;
    if (cols_done == NB) {
      rc = gemm_lower<T>(s, 0, 1, nt, 2 * NB, T(-1), ws.vc + pe, ldw, ws.w + pe, ldw, T(1), A + pe + (int64_t)pe * lda,
                         lda);
      if (rc) return rc;
    } else {
      rc = gemm_lower<T>(s, 0, 1, nt, cols_done, T(-1), ws.vc + pe, ldw, ws.w + pe, ldw, T(1),
                         A + pe + (int64_t)pe * lda, lda);
      if (rc) return rc;
      rc = gemm_lower<T>(s, 0, 1, nt, cols_done, T(-1), ws.w + pe, ldw, ws.vc + pe, ldw, T(1),
                         A + pe + (int64_t)pe * lda, lda);
      if (rc) return rc;
    }
  }
  return kOk;
}

}  // namespace soapmi
