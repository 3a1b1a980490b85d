// Two-stage tridiagonalisation of a dense symmetric matrix, the alternative to sytrd.hpp behind the
// same eigensolver entry points (the analogue of ELPA's two-stage solver; the reference fixes the
// one-stage one at src/soap_tp/csrc/elpa_bindings.cpp:149).
//
//   stage 1  dense -> band (half bandwidth kSbNb = 32): for every panel of 32 columns a Householder
//            QR of the block below the band and a two-sided update of the trailing matrix,
//            A22 <- Q^T A22 Q = A22 - V Y^T - Y V^T with X = A22 V T, Y = X - 1/2 V T^T (V^T X).
//            All of the n^3-order work runs on the MFMA product and the trailing matrix is read
//            twice per 32 columns, not once per column as in the one-stage reduction.
//   stage 2  band -> tridiagonal by bulge chasing: sweep s annihilates column s below the first
//            subdiagonal with a reflector of length <= 32 and chases the bulge this creates down the
//            band, 32 rows per task.  Task (s, k) depends on (s, k-1) and (s-1, k+1), so all tasks
//            with 2 s + k = t are independent: one launch per t, one wavefront per task, blocks in LDS.
//   back 2   Z <- Q2 Z: the stage-2 reflectors of 32 consecutive sweeps at one position form a
//            63 x 32 parallelogram that is applied as one compact-WY block; blocks of sweep group i at
//            position k commute with all blocks that share their "time" 2 (groups - 1 - i) + k, so
//            every time step is one launch over (blocks of the step) x (column chunks), on the
//            transposed eigenvector matrix; in fp64 the three products of a block run on the matrix
//            cores with the window held in registers.
//   back 1   Z <- Q1 Z with the stage-1 reflectors, 256 columns per compact-WY block.
#pragma once
#include "common.hpp"
#include "elementwise.hpp"
#include "gemm.hpp"
#include "qr.hpp"

namespace soapmi {

constexpr int kSbNb = 32;          // half bandwidth of the intermediate band matrix
constexpr int kSbLd = 2 * kSbNb;   // rows of the band storage: AB[i - j + kSbLd * j] = A[i, j], j <= i < j + 2 b
constexpr int kSbBlockStride = 2 * 32 * 32;  // per stage-2 block: V in compact form (32 x 32) and T (32 x 32)

template <typename T>
struct TwoStageWorkspace {
  T* tau1;   // n            stage-1 reflector scalars, by column
  T* part;   // 2 x nwg x 32 partial sums of the panel factorisation
  T* piv;    // 2 x 32
  T* p3;     // n x 96       [V | Y | V] of the current panel
  T* wt;     // 32 x n       V^T A22
  T* xt;     // 32 x n       X^T, then Y^T
  T* small;  // 2 x 32 x 32
  T* ab;     // 64 x n       band matrix
  T* vv;     // n x n        stage-2 reflectors: column s holds the reflectors of sweep s end to end
  T* tau2;   // kmax x n     tau2[k * n + s]
  T* zpad;   // (n + 64) x n eigenvectors, column-major with leading dimension ldz = n + 64
  T* zt;     // n x (n + 64)  their transpose with 64 zero rows below, so that every 63-row window exists
  T* blk;    // all stage-2 blocks x kSbBlockStride
  int64_t ldz;
};

static inline int64_t sb_block_count(int64_t n);

template <typename T>
__global__ void fill_zero_wide_kernel(T* __restrict__ p, int64_t count) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < count; i += (int64_t)gridDim.x * blockDim.x)
    p[i] = T(0);
}

template <typename T, class WS>
static inline void two_stage_workspace_layout(WS& ws, int64_t n, TwoStageWorkspace<T>* out) {
  TwoStageWorkspace<T> w;
  const int64_t nwg = ceil_div64(n, 256);
  const int64_t kmax = n / kSbNb + 2;
  w.ldz = n + 64;
  w.tau1 = ws.template take<T>((size_t)n);
  w.part = ws.template take<T>((size_t)2 * nwg * kQrNb);
  w.piv = ws.template take<T>(2 * kQrNb);
  w.p3 = ws.template take<T>((size_t)n * 96);
  w.wt = ws.template take<T>((size_t)n * 32);
  w.xt = ws.template take<T>((size_t)n * 32);
  w.small = ws.template take<T>(2 * 32 * 32);
  w.ab = ws.template take<T>((size_t)kSbLd * n);
  w.vv = ws.template take<T>((size_t)n * n);
  w.tau2 = ws.template take<T>((size_t)kmax * n);
  w.zpad = ws.template take<T>((size_t)w.ldz * n);
  w.zt = ws.template take<T>((size_t)w.ldz * n);
  w.blk = ws.template take<T>((size_t)sb_block_count(n) * kSbBlockStride);
  if (out) *out = w;
}

// ---- stage 1 ---------------------------------------------------------------------------------

// AB <- the band of A (lower part, i - j <= b), rows b + 1 .. 2 b - 1 of the storage zero.
template <typename T>
__global__ void sb_pack_band_kernel(const T* __restrict__ A, int64_t lda, int n, T* __restrict__ AB) {
  const int j = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int l = threadIdx.x & 63;
  if (j >= n) return;
  const int i = j + l;
  AB[l + (int64_t)kSbLd * j] = (l <= kSbNb && i < n) ? A[i + (int64_t)j * lda] : T(0);
}

template <typename T>
__global__ void sb_extract_tridiagonal_kernel(const T* __restrict__ AB, int n, T* __restrict__ d, T* __restrict__ e) {
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= n) return;
  d[j] = AB[(int64_t)kSbLd * j];
  if (j + 1 < n) e[j] = AB[1 + (int64_t)kSbLd * j];
}

// Y (rows x nbw, ld ldy) <- the transpose of yt (nbw x rows, ld 32), with its first `lead` rows zero.
template <typename T>
__global__ void sb_form_y_kernel(const T* __restrict__ yt, T* __restrict__ Y, int64_t ldy, int nbw, int rows, int lead) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= rows) return;
  for (int c = 0; c < nbw; ++c) Y[r + (int64_t)c * ldy] = (r < lead) ? T(0) : yt[c + 32 * (int64_t)r];
}

// A (n x n, lower triangle referenced) -> band form in place: on exit the band holds Q1^T A Q1
// (lower part), the stage-1 reflectors lie below it (column j: unit entry at row j + b, vector
// below), their scalars in ws.tau1.  The upper triangle of A is used as scratch.
template <typename T>
static inline int sy2sb_lower(hipStream_t s, T* A, int64_t lda, int n, const TwoStageWorkspace<T>& ws,
                              const BlockReflectorWs<T>& br, T* t_block) {
  constexpr int b = kSbNb;
  using Skinny = typename SkinnyTile<T>::type;
  const int np = n - b;  // rows/columns of the matrix seen from one band width down
  if (np <= 0) return kOk;
  {
    const unsigned nb = (unsigned)ceil_div64(n, 64);
    hipLaunchKernelGGL((symmetrize_lower_kernel<T>), dim3(nb, nb), dim3(256), 0, s, A, lda, n);
    SOAPMI_LAUNCH_CHECK();
  }
  T* Ap = A + b;  // Ap[i, j] = A[i + b, j]: the panel of columns [p, pe) has its pivots on Ap's diagonal
  const int64_t ldp = n;
  for (int p = 0; p < np; p += b) {
    const int pe = std::min(np, p + b), nbw = pe - p;
    const int rows = np - p;
    const int nwg = (int)ceil_div64(rows, 256);
    T* part[2] = {ws.part, ws.part + (size_t)nwg * kQrNb};
    T* piv[2] = {ws.piv, ws.piv + kQrNb};
    for (int j = p - 1; j < pe; ++j) {
      const int in = (j - p + 1) & 1, out = in ^ 1;
      hipLaunchKernelGGL((qr_panel_step_kernel<T>), dim3(nwg), dim3(256), 0, s, Ap, lda, np, p, pe, j, part[in], piv[in],
                         part[out], piv[out], ws.tau1, nwg);
    }
    SOAPMI_LAUNCH_CHECK();
    if (rows <= 1) break;  // nothing below: no trailing matrix to update
    // The products below start `lead` rows above the first row the reflectors touch, at a multiple
    // of 128, with V carrying zeros in those rows: for n a multiple of 128 every extent is then a
    // multiple of the MFMA tile and the products take the fast path.
    const int lead = (p + b) % 128;
    const int rows_al = rows + lead;
    const int r_al = p + b - lead;
    // [V | Y | V]: V in the first and the third slot now, Y below
    T* V = ws.p3;
    T* Y = ws.p3 + (int64_t)nbw * ldp;
    T* V2 = ws.p3 + (int64_t)2 * nbw * ldp;
    launch_extract_v<T>(s, Ap, lda, rows_al, p - lead, p, nbw, V, ldp, lead);
    launch_extract_v<T>(s, Ap, lda, rows_al, p - lead, p, nbw, V2, ldp, lead);
    SOAPMI_LAUNCH_CHECK();
    BlockReflectorWs<T> inner = br;
    inner.v = V;
    int rc = build_t_factor<T>(s, inner, rows_al, nbw, ldp, ws.tau1 + p, t_block);
    if (rc) return rc;
    if (nbw < b) {
      // Last block column with fewer rows below the band than columns: the columns [pe, p + b) have no
      // reflector of their own but lie in the rows Q^T acts on: C <- (I - V T^T V^T) C.
      rc = apply_block_reflector<T>(s, inner, t_block, true, rows_al, nbw, p + b - pe, ldp,
                                    A + r_al + (int64_t)pe * lda, lda);
      if (rc) return rc;
    }
    T* A22 = A + r_al + (int64_t)r_al * lda;  // the trailing matrix, extended by `lead` rows and columns
    // wt = V^T A22 (nbw x rows_al); its first `lead` columns belong to no trailing column and are dropped below
    rc = gemm<T, Skinny>(s, 1, 0, nbw, rows_al, rows_al, T(1), V, ldp, A22, lda, T(0), ws.wt, 32,
                         split_count(ceil_div64(rows_al, Skinny::BN), rows_al, nbw, rows_al, ldp), br.splitk);
    if (rc) return rc;
    // xt = T^T wt = X^T
    rc = gemm<T>(s, 1, 0, nbw, rows_al, nbw, T(1), t_block, kBrMax, ws.wt, 32, T(0), ws.xt, 32);
    if (rc) return rc;
    // small0 = X^T V = (V^T X)^T ; small1 = small0 T
    T* s0 = ws.small;
    T* s1 = ws.small + 32 * 32;
    rc = gemm<T, Skinny>(s, 0, 0, nbw, nbw, rows_al, T(1), ws.xt, 32, V, ldp, T(0), s0, 32,
                         split_count(1, rows_al, nbw, nbw, ldp), br.splitk);
    if (rc) return rc;
    rc = gemm<T>(s, 0, 0, nbw, nbw, nbw, T(1), s0, 32, t_block, kBrMax, T(0), s1, 32);
    if (rc) return rc;
    // xt <- Y^T = X^T - 1/2 (S^T T) V^T
    rc = gemm<T>(s, 0, 1, nbw, rows_al, nbw, T(-0.5), s1, 32, V, ldp, T(1), ws.xt, 32);
    if (rc) return rc;
    hipLaunchKernelGGL((sb_form_y_kernel<T>), dim3((unsigned)ceil_div64(rows_al, 256)), dim3(256), 0, s, ws.xt, Y, ldp,
                       nbw, rows_al, lead);
    SOAPMI_LAUNCH_CHECK();
    // A22 -= [V | Y] [Y | V]^T
    rc = gemm<T>(s, 0, 1, rows_al, rows_al, 2 * nbw, T(-1), V, ldp, Y, ldp, T(1), A22, lda);
    if (rc) return rc;
  }
  return kOk;
}

// ---- stage 2 ---------------------------------------------------------------------------------

template <typename T>
__device__ __forceinline__ T sb_wave_sum(T v) {
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) v += __shfl_xor(v, m, 64);
  return v;
}
template <typename T>
__device__ __forceinline__ T sb_wave_max(T v) {
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) v = fmax(v, __shfl_xor(v, m, 64));
  return v;
}

// Householder vector of x (entry i in lane i < len of the lower half-wavefront, zero elsewhere):
// (I - tau v v^T) x = beta e_0 with v_0 = 1, LAPACK's sign convention; the vector is scaled by its
// largest magnitude first, so that neither tiny nor huge entries spoil the norm.
template <typename T>
__device__ __forceinline__ void sb_make_reflector(T x, int lane, int len, T* v, T* tau, T* beta) {
  const bool tail = lane >= 1 && lane < len;
  const T alpha = __shfl(x, 0, 64);
  const T biggest = sb_wave_max<T>(tail ? fabs(x) : T(0));
  if (!(biggest > T(0))) {  // nothing to annihilate (or NaN): the identity
    *tau = T(0);
    *beta = alpha;
    *v = (lane == 0) ? T(1) : T(0);
    return;
  }
  const T unit = fmax(biggest, fabs(alpha));
  const T xs = (lane < len) ? x / unit : T(0);
  const T as = alpha / unit;
  const T tail2 = sb_wave_sum<T>(tail ? xs * xs : T(0));
  const T nrm = sqrt(as * as + tail2);
  const T bs = (as >= T(0)) ? -nrm : nrm;
  *tau = (bs - as) / bs;
  *beta = bs * unit;
  const T inv = T(1) / (as - bs);
  *v = (lane == 0) ? T(1) : (tail ? xs * inv : T(0));
}

// D (len x len, symmetric, full storage in LDS at Dm[col * 33 + row]) <- H D H with H = I - tau v v^T,
// v in vs[] (LDS).  One wavefront; lane = (half, i): row i, columns of parity `half`.
template <typename T>
__device__ __forceinline__ void sb_two_sided(T* Dm, const T* vs, T* ws, T tau, int lane) {
  const int i = lane & 31, half = lane >> 5;
  T acc = T(0);
#pragma unroll 4
  for (int j = half; j < 32; j += 2) acc += Dm[j * 33 + i] * vs[j];
  acc += __shfl_xor(acc, 32, 64);
  T w = tau * acc;
  const T vi = vs[i];
  const T dot = sb_wave_sum<T>(half == 0 ? w * vi : T(0));
  w -= T(0.5) * tau * dot * vi;
  if (half == 0) ws[i] = w;
  __syncthreads();
#pragma unroll 4
  for (int j = half; j < 32; j += 2) Dm[j * 33 + i] -= vi * ws[j] + w * vs[j];
  __syncthreads();
}

// One launch = all tasks (s, k) with 2 s + k = t.  Workgroup q takes sweep s_hi - q.
template <typename T>
__global__ __launch_bounds__(64) void sb_chase_kernel(T* __restrict__ AB, int n, int t, int s_hi, T* __restrict__ VV,
                                                      int64_t ldvv, T* __restrict__ tau2) {
  constexpr int b = kSbNb;
  __shared__ T Bm[32 * 33];
  __shared__ T Dm[32 * 33];
  __shared__ T vp[32];  // previous reflector of the sweep
  __shared__ T vn[32];  // the new one
  __shared__ T us[32];
  const int lane = threadIdx.x, i = lane & 31, half = lane >> 5;
  const int s = s_hi - (int)blockIdx.x;
  if (s < 0) return;
  const int k = t - 2 * s;
  if (k > (n - 2 - s) / b) return;
  for (int e = lane; e < 32 * 33; e += 64) {
    Bm[e] = T(0);
    Dm[e] = T(0);
  }
  __syncthreads();
  int row0, len;  // the diagonal block this task updates from both sides: rows/columns row0 .. row0 + len - 1
  T x = T(0);
  T tau_p = T(0);
  if (k == 0) {
    row0 = s + 1;
    len = min(b, n - 1 - s);
    if (half == 0 && i < len) x = AB[1 + i + (int64_t)kSbLd * s];
  } else {
    const int st = s + 1 + (k - 1) * b;  // previous reflector: rows st .. st + b - 1
    row0 = st + b;
    len = min(b, n - row0);
    if (half == 0) vp[i] = VV[st + i + (int64_t)s * ldvv];
    tau_p = tau2[(int64_t)(k - 1) * n + s];
    // B[i][j] = A[row0 + i, st + j] = AB[b + i - j, st + j]
    if (i < len)
      for (int j = half; j < b; j += 2) Bm[j * 33 + i] = AB[b + i - j + (int64_t)kSbLd * (st + j)];
  }
  // D[i][j] = A[row0 + i, row0 + j], lower part stored: AB[i - j, row0 + j]
  if (i < len)
    for (int j = half; j <= i; j += 2) {
      const T v = AB[i - j + (int64_t)kSbLd * (row0 + j)];
      Dm[j * 33 + i] = v;
      Dm[i * 33 + j] = v;
    }
  __syncthreads();
  if (k > 0) {
    // B <- B (I - tau_p vp vp^T)
    T acc = T(0);
#pragma unroll 4
    for (int j = half; j < b; j += 2) acc += Bm[j * 33 + i] * vp[j];
    acc += __shfl_xor(acc, 32, 64);
    const T u = tau_p * acc;
#pragma unroll 4
    for (int j = half; j < b; j += 2) Bm[j * 33 + i] -= u * vp[j];
    __syncthreads();
    x = (half == 0 && i < len) ? Bm[i] : T(0);  // first column of B: the bulge
  }
  T v, tau, beta;
  {
    T v_low;  // defined in the lower half-wavefront only
    sb_make_reflector<T>(x, lane, len, &v_low, &tau, &beta);
    if (half == 0) vn[i] = v_low;
  }
  if (k == 0) {
    if (half == 0 && i < len) AB[1 + i + (int64_t)kSbLd * s] = (i == 0) ? beta : T(0);
    __syncthreads();
    v = vn[i];
  } else {
    if (half == 0) Bm[i] = (i == 0) ? beta : T(0);
    __syncthreads();
    v = vn[i];
    // columns 1 .. b-1 of B <- (I - tau v v^T) B
    {
      const int j = i;  // lane (half, j): column j, rows of parity `half`
      T z = T(0);
#pragma unroll 4
      for (int r = half; r < 32; r += 2) z += vn[r] * Bm[j * 33 + r];
      z += __shfl_xor(z, 32, 64);
      if (half == 0) us[j] = (j >= 1) ? tau * z : T(0);
    }
    __syncthreads();
#pragma unroll 4
    for (int j = half; j < b; j += 2) Bm[j * 33 + i] -= v * us[j];
    __syncthreads();
    const int st = s + 1 + (k - 1) * b;
    if (i < len)
      for (int j = half; j < b; j += 2) AB[b + i - j + (int64_t)kSbLd * (st + j)] = Bm[j * 33 + i];
  }
  sb_two_sided<T>(Dm, vn, us, tau, lane);
  if (i < len)
    for (int j = half; j <= i; j += 2) AB[i - j + (int64_t)kSbLd * (row0 + j)] = Dm[j * 33 + i];
  if (half == 0 && i < len) VV[row0 + i + (int64_t)s * ldvv] = v;
  if (lane == 0) tau2[(int64_t)k * n + s] = tau;
}

template <typename T>
static inline int sb2st(hipStream_t s, int n, const TwoStageWorkspace<T>& ws, T* d, T* e) {
  constexpr int b = kSbNb;
  if (n >= 3) {
    const int kcap = (n - 2) / b;
    for (int t = 0; t <= 2 * n - 6; ++t) {
      const int s_hi = std::min(n - 3, t / 2);
      const int grid = std::min(s_hi + 1, kcap / 2 + 1);
      hipLaunchKernelGGL((sb_chase_kernel<T>), dim3(grid), dim3(64), 0, s, ws.ab, n, t, s_hi, ws.vv, (int64_t)n, ws.tau2);
    }
    SOAPMI_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL((sb_extract_tridiagonal_kernel<T>), dim3((unsigned)ceil_div64(n, 256)), dim3(256), 0, s, ws.ab, n, d, e);
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

// ---- back-transformation of stage 2 -------------------------------------------------------------

// Number of stage-2 blocks (sweep group, position): group gi has positions 0 .. K0 - gi, K0 = (n - 2) / b.
static inline int64_t sb_block_count(int64_t n) {
  if (n < 3) return 0;
  const int64_t groups = ceil_div64(n - 2, kSbNb), k0 = (n - 2) / kSbNb;
  return groups * (k0 + 1) - groups * (groups - 1) / 2;
}
__host__ __device__ __forceinline__ int64_t sb_block_index(int gi, int k, int k0) {
  return (int64_t)gi * (k0 + 1) - (int64_t)gi * (gi - 1) / 2 + k;
}

// Block (gi, k): the reflectors of sweeps 32 gi .. 32 gi + 31 at position k.  Column c of the block
// has its unit entry in row c of the block's 63-row window and 32 entries in all, so the block is
// stored compactly: Vc[l + 32 c] = V[c + l][c], followed by the compact-WY factor T (32 x 32, ld 32).
template <typename T>
__global__ __launch_bounds__(256) void sb_build_blocks_kernel(const T* __restrict__ VV, int64_t ldvv,
                                                              const T* __restrict__ tau2, int n, T* __restrict__ blk) {
  constexpr int b = kSbNb, g = kSbNb;
  __shared__ T Vs[32][65];  // Vs[c][r]: full 63-row window, zero outside the parallelogram
  __shared__ T Gs[32][33];
  __shared__ T Ts[32][33];
  __shared__ T taus[32];
  const int tid = threadIdx.x;
  const int gi = blockIdx.x, k = blockIdx.y;
  const int k0 = (n - 2) / b;
  if (k > k0 - gi) return;
  const int s0 = gi * g;
  const int nsw = n - 2;
  T* out = blk + sb_block_index(gi, k, k0) * kSbBlockStride;
  for (int e = tid; e < 32 * 65; e += 256) (&Vs[0][0])[e] = T(0);
  __syncthreads();
  {
    const int c = tid >> 3, part = tid & 7;  // 8 threads per column, 4 entries each
    const int sw = s0 + c;
    const bool exists = sw < nsw && k <= (n - 2 - sw) / b;
    if (exists) {
      const int st = sw + 1 + k * b;
      const int len = min(b, n - st);
      for (int l = part * 4; l < part * 4 + 4; ++l)
        if (l < len) Vs[c][c + l] = VV[st + l + (int64_t)sw * ldvv];
    }
    if (part == 0) taus[c] = exists ? tau2[(int64_t)k * n + sw] : T(0);
  }
  __syncthreads();
  for (int e = tid; e < 32 * 32; e += 256) {
    const int a = e & 31, c = e >> 5;
    T sum = T(0);
#pragma unroll 8
    for (int r = 0; r < 64; ++r) sum += Vs[a][r] * Vs[c][r];
    Gs[a][c] = sum;
  }
  __syncthreads();
  if (tid < 32) {
    const int a = tid;  // row a of T: T[a][c] = -tau_c sum_{l=a}^{c-1} T[a][l] G[l][c] for c > a
    for (int c = 0; c < 32; ++c) {
      T value = T(0);
      if (c == a) value = taus[c];
      else if (c > a) {
        T sum = T(0);
        for (int l = a; l < c; ++l) sum += Ts[a][l] * Gs[l][c];
        value = -taus[c] * sum;
      }
      Ts[a][c] = value;
    }
  }
  __syncthreads();
  for (int e = tid; e < 32 * 32; e += 256) {
    const int l = e & 31, c = e >> 5;
    out[e] = Vs[c][c + l];
    out[32 * 32 + e] = Ts[l][c];  // T[a = l][c] at a + 32 c
  }
}

// One time step of the back-transformation on the transposed eigenvector matrix Zt (element
// (row r, column c) at Zt[c + r * ldt], so that a thread per column reads coalesced): block z of
// the step owns the 63 rows from row_first - 96 z and applies (I - V T V^T) to them.  The block's V
// and T are read through LDS at wavefront-uniform addresses; a thread keeps its column of the
// window in registers.
template <typename T>
__global__ __launch_bounds__(256) void sb_apply_blocks_kernel(const T* __restrict__ blk, int n, int t, int ri_lo,
                                                              int groups, T* __restrict__ Zt, int64_t ldt) {
  constexpr int b = kSbNb, g = kSbNb;
  __shared__ T Vc[32 * 32];  // Vc[l + 32 a] = V[a + l][a]
  __shared__ T Tm[32 * 32];  // Tm[a + 32 c]
  const int tid = threadIdx.x;
  const int ri = ri_lo + (int)blockIdx.x;
  const int gi = groups - 1 - ri, k = t - 2 * ri;
  const int k0 = (n - 2) / b;
  const T* src = blk + sb_block_index(gi, k, k0) * kSbBlockStride;
  for (int e = tid; e < 32 * 32; e += 256) {
    Vc[e] = src[e];
    Tm[e] = src[32 * 32 + e];
  }
  __syncthreads();
  const int col = blockIdx.y * 256 + tid;
  if (col >= n) return;
  const int64_t r0 = (int64_t)gi * g + 1 + (int64_t)k * b;
  T* zp = Zt + col + r0 * ldt;
  T z[63];
#pragma unroll
  for (int r = 0; r < 63; ++r) z[r] = zp[(int64_t)r * ldt];
  // The loops are unrolled in full (every register index is a compile-time constant); the scheduling
  // barriers keep the compiler from hoisting all the LDS reads of the unrolled code to the front,
  // which would need thousands of registers.
  T w[32];
#pragma unroll
  for (int a = 0; a < 32; ++a) {
    T sum = T(0);
#pragma unroll
    for (int l = 0; l < 32; ++l) sum += Vc[l + 32 * a] * z[a + l];
    w[a] = sum;
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int a = 0; a < 32; ++a) {  // w <- T w, T upper triangular: entry a needs entries a .. 31 only
    T sum = T(0);
#pragma unroll
    for (int c = a; c < 32; ++c) sum += Tm[a + 32 * c] * w[c];
    w[a] = sum;
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int a = 0; a < 32; ++a) {
#pragma unroll
    for (int l = 0; l < 32; ++l) z[a + l] -= Vc[l + 32 * a] * w[a];
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int r = 0; r < 63; ++r) zp[(int64_t)r * ldt] = z[r];
}

// The same time step on the fp64 matrix cores.  A wavefront owns 64 columns of the block's 64-row
// window (the 63 rows the block touches and one more, whose row of V is zero) and keeps them in the
// "b" operand layout of v_mfma_f64_16x16x4: register (ks, ct) of lane l holds row 4 ks + l / 16 of
// column 16 ct + l % 16.  That is also the accumulator layout of the 16-row tile ks / 4, register
// ks % 4, so the three products chain without a layout change:
//   W  = V^T Z   "a" = pieces of V^T from LDS, "b" = the window registers
//   W2 = T W     "a" = pieces of T,            "b" = W's accumulator registers (register r = k step r)
//   Z -= V W2    "a" = pieces of -V,           "b" = W2's registers, accumulated onto the window registers
// Tiles of V that lie outside the parallelogram are skipped: columns 16 j .. 16 j + 15 of V have
// their entries in rows 16 j .. 16 j + 46 only.
__global__ __launch_bounds__(256) void sb_apply_blocks_mfma_kernel(const double* __restrict__ blk, int n, int t,
                                                                  int ri_lo, int groups, double* __restrict__ Zt,
                                                                  int64_t ldt) {
  constexpr int b = kSbNb, g = kSbNb;
  using MF = Mfma<double>;
  __shared__ double Vd[64 * 32];  // Vd[r * 32 + a] = V[r][a]
  __shared__ double Vn[32 * 64];  // Vn[a * 64 + r] = -V[r][a]
  __shared__ double Tt[32 * 32];  // Tt[c * 32 + a] = T[a][c]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ri = ri_lo + (int)blockIdx.x;
  const int gi = groups - 1 - ri, k = t - 2 * ri;
  const int k0 = (n - 2) / b;
  const double* src = blk + sb_block_index(gi, k, k0) * kSbBlockStride;
  for (int e = tid; e < 64 * 32; e += 256) {
    Vd[e] = 0.0;
    Vn[e] = 0.0;
  }
  __syncthreads();
  for (int e = tid; e < 32 * 32; e += 256) {
    const int l = e & 31, a = e >> 5;  // compact form: src[l + 32 a] = V[a + l][a]
    const double v = src[e];
    Vd[(a + l) * 32 + a] = v;
    Vn[a * 64 + a + l] = -v;
    Tt[e] = src[32 * 32 + e];  // stored as T[a][c] at a + 32 c already
  }
  __syncthreads();
  const int c0 = (blockIdx.y * 4 + wave) * 64;  // this wavefront's first column
  if (c0 >= n) return;
  const int64_t r0 = (int64_t)gi * g + 1 + (int64_t)k * b;
  const int kq = lane >> 4, idx = lane & 15;
  double* zp = Zt + c0 + idx + (r0 + kq) * ldt;  // + 16 ct + 4 ks ldt
  // columns beyond n: clamp the address (loads) and skip the store
  bool live[4];
#pragma unroll
  for (int ct = 0; ct < 4; ++ct) live[ct] = c0 + 16 * ct + idx < n;
  MF::Acc z[4][4];  // z[rt][ct][q]: row 16 rt + 4 q + kq, column 16 ct + idx
#pragma unroll
  for (int rt = 0; rt < 4; ++rt)
#pragma unroll
    for (int ct = 0; ct < 4; ++ct)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        z[rt][ct][q] = live[ct] ? zp[16 * ct + (int64_t)(16 * rt + 4 * q) * ldt] : 0.0;
  // W[i][ct] = sum over the rows of V's column tile i: k steps 4 i .. 4 i + 11
  MF::Acc w[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int ct = 0; ct < 4; ++ct)
#pragma unroll
      for (int q = 0; q < 4; ++q) w[i][ct][q] = 0.0;
#pragma unroll
    for (int ks = 4 * i; ks < 4 * i + 12; ++ks) {
      const double a = Vd[(4 * ks + kq) * 32 + 16 * i + idx];  // V^T[a = 16 i + idx][r = 4 ks + kq]
#pragma unroll
      for (int ct = 0; ct < 4; ++ct) w[i][ct] = MF::mma(a, z[ks >> 2][ct][ks & 3], w[i][ct]);
    }
  }
  // W2 = T W, T upper triangular: tile row 0 needs W's tiles 0 and 1, tile row 1 only tile 1
  MF::Acc w2[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int ct = 0; ct < 4; ++ct)
#pragma unroll
      for (int q = 0; q < 4; ++q) w2[i][ct][q] = 0.0;
#pragma unroll
    for (int j = i; j < 2; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const double a = Tt[(16 * j + 4 * q + kq) * 32 + 16 * i + idx];  // T[16 i + idx][16 j + 4 q + kq]
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) w2[i][ct] = MF::mma(a, w[j][ct][q], w2[i][ct]);
      }
    }
  }
  // Z -= V W2: row tile rt of V has entries in column tiles j with rt - 2 <= j <= rt
#pragma unroll
  for (int rt = 0; rt < 4; ++rt) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if (j > rt || j < rt - 2) continue;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const double a = Vn[(16 * j + 4 * q + kq) * 64 + 16 * rt + idx];  // -V[16 rt + idx][16 j + 4 q + kq]
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) z[rt][ct] = MF::mma(a, w2[j][ct][q], z[rt][ct]);
      }
    }
  }
#pragma unroll
  for (int rt = 0; rt < 4; ++rt)
#pragma unroll
    for (int ct = 0; ct < 4; ++ct)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (live[ct]) zp[16 * ct + (int64_t)(16 * rt + 4 * q) * ldt] = z[rt][ct][q];
}

template <typename T>
static inline void launch_apply_blocks(hipStream_t s, const T* blk, int n, int t, int ri_lo, int groups, int count, T* Zt,
                                       int64_t ldt) {
  if constexpr (std::is_same<T, double>::value) {
    hipLaunchKernelGGL(sb_apply_blocks_mfma_kernel, dim3(count, (unsigned)ceil_div64(n, 256)), dim3(256), 0, s, blk, n, t,
                       ri_lo, groups, Zt, ldt);
  } else {
    hipLaunchKernelGGL((sb_apply_blocks_kernel<T>), dim3(count, (unsigned)ceil_div64(n, 256)), dim3(256), 0, s, blk, n, t,
                       ri_lo, groups, Zt, ldt);
  }
}

// Z (rows 0 .. n-1 of the padded matrix ws.zpad, ld ws.ldz, n columns) <- Q2 Z.  Works on the
// transpose (ws.zt) and writes the result back into ws.zpad.
template <typename T>
static inline int sb_apply_q2(hipStream_t s, int n, const TwoStageWorkspace<T>& ws) {
  constexpr int b = kSbNb, g = kSbNb;
  const int nsw = n - 2;
  if (nsw <= 0) return kOk;
  const int groups = (int)ceil_div64(nsw, g);
  const int k0 = (n - 2) / b;
  hipLaunchKernelGGL((sb_build_blocks_kernel<T>), dim3(groups, k0 + 1), dim3(256), 0, s, ws.vv, (int64_t)n, ws.tau2, n,
                     ws.blk);
  SOAPMI_LAUNCH_CHECK();
  // zt[c + r * n] = zpad[r + c * ldz] for r < n; the 64 rows below stay zero
  const int64_t ldt = n;
  hipLaunchKernelGGL((fill_zero_wide_kernel<T>), dim3(256), dim3(256), 0, s, ws.zt + (int64_t)n * ldt, (int64_t)64 * ldt);
  hipLaunchKernelGGL((transpose_kernel<T>), dim3((unsigned)ceil_div64(n, 64), (unsigned)ceil_div64(n, 64)), dim3(256), 0, s,
                     ws.zpad, ws.ldz, ws.zt, ldt, n, n, transpose_vec_ok<T>(ws.zpad, ws.ldz, ws.zt, ldt, n, n));
  SOAPMI_LAUNCH_CHECK();
  const int t_last = 2 * (groups - 1) + k0;
  for (int t = 0; t <= t_last; ++t) {
    // blocks of this step: ri in [ri_lo, ri_hi], k = t - 2 ri must not exceed k0 - gi = k0 - (groups - 1 - ri)
    const int ri_hi = std::min(groups - 1, t / 2);
    // t - 2 ri <= k0 - groups + 1 + ri  <=>  3 ri >= t - k0 + groups - 1
    const int bound = t - k0 + groups - 1;
    const int ri_lo = std::max(0, bound <= 0 ? 0 : (bound + 2) / 3);
    const int count = ri_hi - ri_lo + 1;
    if (count <= 0) continue;
    launch_apply_blocks<T>(s, ws.blk, n, t, ri_lo, groups, count, ws.zt, ldt);
  }
  SOAPMI_LAUNCH_CHECK();
  hipLaunchKernelGGL((transpose_kernel<T>), dim3((unsigned)ceil_div64(n, 64), (unsigned)ceil_div64(n, 64)), dim3(256), 0, s,
                     ws.zt, ldt, ws.zpad, ws.ldz, n, n, transpose_vec_ok<T>(ws.zt, ldt, ws.zpad, ws.ldz, n, n));
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

// Z (rows 0 .. n-1 of the padded matrix) <- Q1 Z with the stage-1 reflectors left below the band of A.
template <typename T>
static inline int sb_apply_q1(hipStream_t s, const T* A, int64_t lda, int n, const TwoStageWorkspace<T>& ws,
                              const BlockReflectorWs<T>& br, T* t_block) {
  constexpr int b = kSbNb, OB = kBrMax;
  const int np = n - b;
  if (np <= 0) return kOk;
  const T* Ap = A + b;
  const int64_t ldv = n;
  const int blocks = (int)ceil_div64(np, OB);
  for (int bi = blocks - 1; bi >= 0; --bi) {
    const int P = bi * OB, PE = std::min(np, P + OB), nbw = PE - P;
    const int rows = np - P;
    launch_extract_v<T>(s, Ap, lda, rows, P, P, nbw, br.v, ldv);
    SOAPMI_LAUNCH_CHECK();
    int rc = build_t_factor<T>(s, br, rows, nbw, ldv, ws.tau1 + P, t_block);
    if (rc) return rc;
    rc = apply_block_reflector<T>(s, br, t_block, false, rows, nbw, n, ldv, ws.zpad + (P + b), ws.ldz);
    if (rc) return rc;
  }
  return kOk;
}

}  // namespace soapmi
