// Blocked Householder QR (LAPACK geqrf sign convention) and explicit formation of Q, for the
// power-iteration refresh of a SOAP eigenbasis (what the reference obtains from SLATE's
// geqrf + unmqr on the identity: src/soap_tp/csrc/slate_bindings.cpp:176-185).
//
// Panel (NB = 32 columns): one launch per column.  A workgroup owns 256 rows, one per thread,
// and keeps its row of the panel in registers.  Launch j applies reflector j (whose dot
// products with the remaining panel columns were reduced by launch j-1) and, in the same pass,
// reduces the dot products reflector j+1 needs: a 32-value butterfly over the wavefront, then
// a fixed-order sum over workgroups.  No atomics, so results do not depend on scheduling.
// Trailing matrix and Q formation: compact-WY block reflectors on the MFMA GEMM.
#pragma once
#include "common.hpp"
#include "gemm.hpp"

namespace soapmi {

constexpr int kQrNb = 32;

// After the call lane l holds, in the return value, the sum over the wavefront of vals[(l>>1)&31].
template <typename T>
__device__ __forceinline__ T wave_reduce_32(T (&vals)[32], int lane) {
#pragma unroll
  for (int half = 16, mask = 32; half >= 1; half >>= 1, mask >>= 1) {
    const bool upper = (lane & mask) != 0;
#pragma unroll
    for (int c = 0; c < half; ++c) {
      const T send = upper ? vals[c] : vals[c + half];
      const T keep = upper ? vals[c + half] : vals[c];
      vals[c] = keep + __shfl_xor(send, mask, 64);
    }
  }
  return vals[0] + __shfl_xor(vals[0], 1, 64);
}

template <typename T>
__global__ __launch_bounds__(256) void qr_panel_step_kernel(T* __restrict__ A, int64_t lda, int n, int p, int pe, int j,
                                                            const T* __restrict__ part_in,
                                                            const T* __restrict__ piv_in, T* __restrict__ part_out,
                                                            T* __restrict__ piv_out, T* __restrict__ tau, int nwg) {
  constexpr int NB = kQrNb;
  __shared__ T s_dots[NB];
  __shared__ T s_tc[NB];
  __shared__ T s_wave[4][NB];
  __shared__ T s_scal[3];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = p + blockIdx.x * 256 + tid;
  const bool apply = (j >= p);
  const int c0 = apply ? j : p;  // first panel column held in registers
  const int ncol = pe - c0;
  const bool live = r < n;

  T a[NB];
#pragma unroll
  for (int c = 0; c < NB; ++c) a[c] = (live && c < ncol) ? A[r + (int64_t)(c0 + c) * lda] : T(0);

  if (apply) {
    if (tid < ncol) {
      T s = T(0);
      for (int w = 0; w < nwg; ++w) s += part_in[w * NB + tid];
      s_dots[tid] = s;
    }
    __syncthreads();
    if (tid == 0) {
      const T alpha = piv_in[0];
      const T x2 = s_dots[0];
      T beta = alpha, tauv = T(0), scale = T(0);
      if (x2 > T(0)) {
        const T nrm = sqrt(alpha * alpha + x2);
        beta = (alpha >= T(0)) ? -nrm : nrm;
        tauv = (beta - alpha) / beta;
        scale = T(1) / (alpha - beta);
      }
      s_scal[0] = scale; s_scal[1] = beta; s_scal[2] = tauv;
    }
    __syncthreads();
    const T scale = s_scal[0], beta = s_scal[1], tauv = s_scal[2];
    if (tid >= 1 && tid < ncol) s_tc[tid] = tauv * (piv_in[tid] + scale * s_dots[tid]);
    __syncthreads();
    if (live && r >= j) {
      if (r > j) {
        const T v = a[0] * scale;
        a[0] = v;
#pragma unroll
        for (int c = 1; c < NB; ++c)
          if (c < ncol) a[c] -= s_tc[c] * v;
      } else {
        a[0] = beta;
#pragma unroll
        for (int c = 1; c < NB; ++c)
          if (c < ncol) a[c] -= s_tc[c];
        tau[j] = tauv;
      }
#pragma unroll
      for (int c = 0; c < NB; ++c)
        if (c < ncol) A[r + (int64_t)(c0 + c) * lda] = a[c];
    }
  }

  const int jn = j + 1;
  if (jn >= pe) return;
  // Column jn sits in a[1] after an apply step, in a[0] on the opening launch of a panel.
  const T an = apply ? a[1] : a[0];
  const bool below = live && r > jn;
  T vals[NB];
#pragma unroll
  for (int c = 0; c < NB; ++c) {
    const T other = apply ? ((c + 1 < NB) ? a[(c + 1) % NB] : T(0)) : a[c];
    vals[c] = below ? an * other : T(0);
  }
  if (live && r == jn) {
#pragma unroll
    for (int c = 0; c < NB; ++c) {
      const T other = apply ? ((c + 1 < NB) ? a[(c + 1) % NB] : T(0)) : a[c];
      if (c < pe - jn) piv_out[c] = other;
    }
  }
  const T total = wave_reduce_32<T>(vals, lane);
  if ((lane & 1) == 0) s_wave[wave][(lane >> 1) & 31] = total;
  __syncthreads();
  if (tid < NB) part_out[blockIdx.x * NB + tid] = s_wave[0][tid] + s_wave[1][tid] + s_wave[2][tid] + s_wave[3][tid];
}

// Vc (nrows x nbw, ld ldv) <- the unit-lower-trapezoidal reflector block stored in A with its
// unit diagonal at (row0 + c, col0 + c): zeros above, ones on, A below.
template <typename T>
__global__ void extract_v_kernel(const T* __restrict__ A, int64_t lda, int nrows, int row0, int col0, int nbw,
                                 T* __restrict__ Vc, int64_t ldv) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;  // row within the block
  if (i >= nrows) return;
  for (int c = 0; c < nbw; ++c) {
    T v;
    if (i < c) v = T(0);
    else if (i == c) v = T(1);
    else v = A[(row0 + i) + (int64_t)(col0 + c) * lda];
    Vc[i + (int64_t)c * ldv] = v;
  }
}

// Compact-WY factor: T upper triangular with H_0 ... H_{nbw-1} = I - V T V^T, from G = V^T V.
// One wavefront; column i needs the finished columns 0..i-1.
template <typename T>
__global__ void larft_kernel(const T* __restrict__ G, int ldg, const T* __restrict__ tau, int nbw, T* __restrict__ Tm,
                             int ldt) {
  __shared__ T t[64][65];
  const int k = threadIdx.x;
  for (int c = 0; c < 64; ++c) t[k][c] = T(0);
  __syncthreads();
  for (int i = 0; i < nbw; ++i) {
    const T ti = tau[i];
    T s = T(0);
    if (k < i) {
      for (int l = k; l < i; ++l) s += t[k][l] * G[l + i * ldg];
      s = -ti * s;
    }
    __syncthreads();
    if (k < i) t[k][i] = s;
    if (k == i) t[i][i] = ti;
    __syncthreads();
  }
  for (int c = 0; c < nbw; ++c)
    if (k < nbw) Tm[k + c * ldt] = t[k][c];
}

// Finishes the panel columns of the explicit Q: rows above the panel are zero and the unit
// diagonal of [I; 0] is added to -V (T V1^T).
template <typename T>
__global__ void orgqr_panel_fix_kernel(T* __restrict__ Q, int64_t ldq, int p, int nbw) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < p) {
    for (int c = 0; c < nbw; ++c) Q[i + (int64_t)(p + c) * ldq] = T(0);
  } else if (i < p + nbw) {
    Q[i + (int64_t)i * ldq] += T(1);
  }
}

template <typename T>
struct QrWorkspace {
  T* vc;      // n x NB
  T* t_all;   // panels x NB x NB
  T* tau;     // n
  T* gram;    // NB x NB
  T* w;       // NB x n
  T* w2;      // NB x n
  T* mx;      // NB x NB
  T* part;    // 2 x nwg x NB
  T* piv;     // 2 x NB
  T* splitk;  // kSplits x NB x n
};
constexpr int kQrSplits = 8;

template <typename T, class WS>
static inline void qr_workspace_layout(WS& ws, int64_t n, QrWorkspace<T>* out) {
  const int64_t panels = ceil_div64(n, kQrNb);
  const int64_t nwg = ceil_div64(n, 256);
  T* vc = ws.template take<T>((size_t)n * kQrNb);
  T* t_all = ws.template take<T>((size_t)panels * kQrNb * kQrNb);
  T* tau = ws.template take<T>((size_t)n);
  T* gram = ws.template take<T>(kQrNb * kQrNb);
  T* w = ws.template take<T>((size_t)n * kQrNb);
  T* w2 = ws.template take<T>((size_t)n * kQrNb);
  T* mx = ws.template take<T>(kQrNb * kQrNb);
  T* part = ws.template take<T>((size_t)2 * nwg * kQrNb);
  T* piv = ws.template take<T>(2 * kQrNb);
  T* splitk = ws.template take<T>((size_t)kQrSplits * kQrNb * n);
  if (out) *out = QrWorkspace<T>{vc, t_all, tau, gram, w, w2, mx, part, piv, splitk};
}

template <typename T>
static inline size_t qr_workspace_bytes(int64_t n) {
  WorkspaceSizer sizer;
  qr_workspace_layout<T>(sizer, n, nullptr);
  return sizer.total();
}

// Applies the block reflector (or its transpose) of one panel to C (rows x nc, ld ldc) in place:
// C <- C - Vc op(T) Vc^T C.
template <typename T>
static inline int apply_block_reflector(hipStream_t s, const QrWorkspace<T>& ws, const T* Tm, bool transT, int rows,
                                        int nbw, int nc, int64_t ldv, T* C, int64_t ldc) {
  using Skinny = typename SkinnyTile<T>::type;
  if (nc <= 0 || rows <= 0) return kOk;
  // W = Vc^T C  (nbw x nc, K = rows): few output tiles, long K -> split-K with fixed-order reduce
  int splits = 1;
  const int64_t tiles = ceil_div64(nc, Skinny::BN);
  if (tiles < 256 && rows >= 2048) splits = (int)std::min<int64_t>(kQrSplits, ceil_div64(512, tiles));
  int rc = gemm<T, Skinny>(s, 1, 0, nbw, nc, rows, T(1), ws.vc, ldv, C, ldc, T(0), ws.w, kQrNb, splits, ws.splitk);
  if (rc) return rc;
  // W2 = op(T) W
  rc = gemm<T, Skinny>(s, transT ? 1 : 0, 0, nbw, nc, nbw, T(1), Tm, kQrNb, ws.w, kQrNb, T(0), ws.w2, kQrNb);
  if (rc) return rc;
  // C -= Vc W2
  return gemm<T>(s, 0, 0, rows, nc, nbw, T(-1), ws.vc, ldv, ws.w2, kQrNb, T(1), C, ldc);
}

// geqrf in place on A (n x n), then the explicit Q into Qout (n x n).  A is destroyed.
template <typename T>
static inline int qr_factor_and_form_q(hipStream_t s, T* A, int64_t lda, T* Qout, int64_t ldq, int n,
                                       const QrWorkspace<T>& ws) {
  using Skinny = typename SkinnyTile<T>::type;
  const int NB = kQrNb;
  const int panels = (int)ceil_div64(n, NB);
  const int64_t ldv = n;
  // ---- factorisation ----
  for (int pi = 0; pi < panels; ++pi) {
    const int p = pi * NB, pe = std::min(n, p + NB), nbw = pe - p;
    const int rows = n - p;
    const int nwg = (int)ceil_div64(rows, 256);
    T* part[2] = {ws.part, ws.part + (size_t)nwg * NB};
    T* piv[2] = {ws.piv, ws.piv + NB};
    for (int j = p - 1; j < pe; ++j) {
      const int in = (j - p + 1) & 1, out = in ^ 1;
      hipLaunchKernelGGL((qr_panel_step_kernel<T>), dim3(nwg), dim3(256), 0, s, A, lda, n, p, pe, j, part[in], piv[in],
                         part[out], piv[out], ws.tau, nwg);
    }
    SOAPMI_LAUNCH_CHECK();
    hipLaunchKernelGGL((extract_v_kernel<T>), dim3((unsigned)ceil_div64(rows, 256)), dim3(256), 0, s, A, lda, rows, p, p, nbw,
                       ws.vc, ldv);
    int splits = rows >= 2048 ? kQrSplits : 1;
    int rc = gemm<T, Skinny>(s, 1, 0, nbw, nbw, rows, T(1), ws.vc, ldv, ws.vc, ldv, T(0), ws.gram, NB, splits, ws.splitk);
    if (rc) return rc;
    T* Tm = ws.t_all + (size_t)pi * NB * NB;
    hipLaunchKernelGGL((larft_kernel<T>), dim3(1), dim3(64), 0, s, ws.gram, NB, ws.tau + p, nbw, Tm, NB);
    SOAPMI_LAUNCH_CHECK();
    // trailing columns: C <- H^T C = C - V T^T V^T C
    rc = apply_block_reflector<T>(s, ws, Tm, true, rows, nbw, n - pe, ldv, A + p + (int64_t)pe * lda, lda);
    if (rc) return rc;
  }
  // ---- explicit Q, panels in reverse ----
  for (int pi = panels - 1; pi >= 0; --pi) {
    const int p = pi * NB, pe = std::min(n, p + NB), nbw = pe - p;
    const int rows = n - p;
    T* Tm = ws.t_all + (size_t)pi * NB * NB;
    hipLaunchKernelGGL((extract_v_kernel<T>), dim3((unsigned)ceil_div64(rows, 256)), dim3(256), 0, s, A, lda, rows, p, p, nbw,
                       ws.vc, ldv);
    SOAPMI_LAUNCH_CHECK();
    // columns to the right already hold Q of the later panels: C <- (I - V T V^T) C
    int rc = apply_block_reflector<T>(s, ws, Tm, false, rows, nbw, n - pe, ldv, Qout + p + (int64_t)pe * ldq, ldq);
    if (rc) return rc;
    // own columns: [I;0] - V (T V1^T)
    rc = gemm<T, Skinny>(s, 0, 1, nbw, nbw, nbw, T(1), Tm, NB, ws.vc, ldv, T(0), ws.mx, NB);
    if (rc) return rc;
    rc = gemm<T>(s, 0, 0, rows, nbw, nbw, T(-1), ws.vc, ldv, ws.mx, NB, T(0), Qout + p + (int64_t)p * ldq, ldq);
    if (rc) return rc;
    hipLaunchKernelGGL((orgqr_panel_fix_kernel<T>), dim3((unsigned)ceil_div64(pe, 256)), dim3(256), 0, s, Qout, ldq, p,
                       nbw);
    SOAPMI_LAUNCH_CHECK();
  }
  return kOk;
}

}  // namespace soapmi
