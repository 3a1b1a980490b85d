// Divide-and-conquer eigensolver for a symmetric tridiagonal matrix (Cuppen's method with the
// deflation rules of LAPACK laed2 and Gu/Eisenstat's recomputed update vector, laed3), second
// stage of the eigensolver that replaces ELPA (src/soap_tp/csrc/elpa_bindings.cpp:165).
//
// The recursion bottoms out at 1x1 blocks, so there is no separate small-matrix solver: level
// t of the tree merges the 2^t pairs of neighbouring blocks [b(t,q), b(t,q+1)), b(t,q) =
// floor(q n / 2^t), and every level is a fixed sequence of batched launches (one slice of the
// grid per merge).  Sizes that depend on the data (number of non-deflated eigenvalues k) stay in
// device memory: kernels and the batched MFMA product read them there, workgroups with
// nothing to do return at once, and the host never synchronises.
//
// Per merge: sort the eigenvalues of the two children (bitonic, batched); deflate (one
// sequential scan, staged through LDS); apply the deflation rotations and gather the surviving
// eigenvector columns; solve the secular equation with a bracketed rational ("middle way")
// iteration that falls back to bisection, one thread per root in small merges and one wavefront
// per root (poles spread over the lanes) in merges of 256 and more; recompute the update vector
// from the roots; form the k x k eigenvector matrix of the rank-one update; multiply (MFMA).  The
// children's eigenvectors are block diagonal, so a surviving column has support in the top rows,
// the bottom rows, or (after a deflation rotation across the children) both: the deflation scan
// records which, the gather packs the top-supported columns for the top rows and the
// bottom-supported ones for the bottom rows, and the product is done as two half-height products
// whose B operand picks the matching rows of the rank-one eigenvector matrix (about half the flops
// of multiplying the zero blocks along).
// Eigenvector columns are not kept in sorted order between levels (the sort permutation is
// recomputed where it is needed); one final sort orders the result.
#pragma once
#include <limits>

#include "common.hpp"
#include "gemm.hpp"

namespace soapmi {

template <typename T>
struct DcWorkspace {
  T* d;      // n   working eigenvalues (scaled)
  T* e;      // n   scaled off-diagonals
  T* z;      // n
  T* dl;     // n   non-deflated eigenvalues (per merge, compact at [lo, lo+k))
  T* wv;     // n   matching z components
  T* dnew;   // n
  T* zhat;   // n
  T* norm_part;  // kDcNormChunks x n   partial squared norms of the rank-one eigenvectors
  T* mu;     // n   root offsets from their origin poles (wavefront-per-root path)
  int* org;  // n   origin pole of each root
  T* rot_c;  // n
  T* rot_s;  // n
  T* skey;   // 4n  sort keys
  T* scal;   // 8   [0] scale
  int* sidx;   // 4n
  int* idx;    // n   column order: non-deflated first, deflated after
  int* rot_a;  // n
  int* rot_b;  // n
  int* kcount; // n   per merge: k, or -1 for a merge with an empty child
  int* nrot;   // n
  int* pos1;   // n   per non-deflated pole: its column among the top-supported ones, or -1
  int* pos2;   // n   the same for the bottom rows
  int* sel1;   // n   per merge, compact at [lo, lo+k1): the poles with support in the top rows
  int* sel2;   // n   the same for the bottom rows
  int* kc1;    // n   per merge: number of top-supported poles
  int* kc2;    // n
  BatchedGemm<T>* batch;  // 2n: two products per merge
  T* X;  // n x n eigenvectors (block diagonal by level)
  T* S;  // n x n secular differences / rank-one eigenvectors
  int64_t ldx, lds;
};

template <typename T, class WS>
static inline void dc_workspace_layout(WS& ws, int64_t n, DcWorkspace<T>* out) {
  DcWorkspace<T> w;
  w.d = ws.template take<T>(n);
  w.e = ws.template take<T>(n);
  w.z = ws.template take<T>(n);
  w.dl = ws.template take<T>(n);
  w.wv = ws.template take<T>(n);
  w.dnew = ws.template take<T>(n);
  w.zhat = ws.template take<T>(n);
  w.norm_part = ws.template take<T>((size_t)32 * n);
  w.mu = ws.template take<T>(n);
  w.org = ws.template take<int>(n);
  w.rot_c = ws.template take<T>(n);
  w.rot_s = ws.template take<T>(n);
  w.skey = ws.template take<T>(4 * n + 8);
  w.scal = ws.template take<T>(8);
  w.sidx = ws.template take<int>(4 * n + 8);
  w.idx = ws.template take<int>(n);
  w.rot_a = ws.template take<int>(n);
  w.rot_b = ws.template take<int>(n);
  w.kcount = ws.template take<int>(n);
  w.nrot = ws.template take<int>(n);
  w.pos1 = ws.template take<int>(n);
  w.pos2 = ws.template take<int>(n);
  w.sel1 = ws.template take<int>(n);
  w.sel2 = ws.template take<int>(n);
  w.kc1 = ws.template take<int>(n);
  w.kc2 = ws.template take<int>(n);
  w.batch = ws.template take<BatchedGemm<T>>(2 * n);
  w.X = ws.template take<T>((size_t)n * n);
  w.S = ws.template take<T>((size_t)n * n);
  w.ldx = n;
  w.lds = n;
  if (out) *out = w;
}

__host__ __device__ __forceinline__ int dc_bound(int t, int q, int n) { return (int)(((int64_t)q * n) >> t); }

struct DcMerge {
  int lo, mid, hi;
  __device__ __forceinline__ bool empty() const { return mid == lo || mid == hi; }
};
__device__ __forceinline__ DcMerge dc_merge(int t, int q, int n) {
  DcMerge m;
  m.lo = dc_bound(t, q, n);
  m.mid = dc_bound(t + 1, 2 * q + 1, n);
  m.hi = dc_bound(t, q + 1, n);
  return m;
}

// ---- set-up --------------------------------------------------------------------------------
template <typename T>
__global__ void dc_scale_kernel(const T* __restrict__ d0, const T* __restrict__ e0, int n, T* __restrict__ scal) {
  __shared__ T red[1024];
  T m = T(0);
  for (int i = threadIdx.x; i < n; i += 1024) {
    m = fmax(m, fabs(d0[i]));
    if (i < n - 1) m = fmax(m, fabs(e0[i]));
  }
  red[threadIdx.x] = m;
  __syncthreads();
  for (int s = 512; s > 0; s >>= 1) {
    if (threadIdx.x < s) red[threadIdx.x] = fmax(red[threadIdx.x], red[threadIdx.x + s]);
    __syncthreads();
  }
  if (threadIdx.x == 0) scal[0] = (red[0] > T(0)) ? red[0] : T(1);
}

// Every boundary is a cut: d[c] loses |e[c-1]| and |e[c]| (rank-one tearing on both sides).
template <typename T>
__global__ void dc_init_kernel(const T* __restrict__ d0, const T* __restrict__ e0, int n, const T* __restrict__ scal,
                               T* __restrict__ d, T* __restrict__ e) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= n) return;
  const T inv = T(1) / scal[0];
  const T el = (c > 0) ? fabs(e0[c - 1] * inv) : T(0);
  const T er = (c < n - 1) ? fabs(e0[c] * inv) : T(0);
  d[c] = d0[c] * inv - el - er;
  e[c] = (c < n - 1) ? e0[c] * inv : T(0);
}

template <typename T>
__global__ void set_identity_kernel(T* __restrict__ X, int64_t ld, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  for (int j = blockIdx.y; j < n; j += gridDim.y) X[i + (int64_t)j * ld] = (i == j) ? T(1) : T(0);
}

// ---- per-level kernels -----------------------------------------------------------------------
// z = (last row of child 1 | sign * first row of child 2) / sqrt(2); sort keys.
template <typename T>
__global__ void dc_z_keys_kernel(int t, int n, int np, const T* __restrict__ X, int64_t ldx, const T* __restrict__ d,
                                 const T* __restrict__ e, T* __restrict__ z, T* __restrict__ skey,
                                 int* __restrict__ sidx) {
  const int q = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= np) return;
  const DcMerge m = dc_merge(t, q, n);
  const int N = m.hi - m.lo;
  const int64_t slot = (int64_t)q * np + c;
  sidx[slot] = c;
  if (m.empty() || c >= N) {
    skey[slot] = std::numeric_limits<T>::infinity();
    return;
  }
  const int g = m.lo + c;
  skey[slot] = d[g];
  const T inv_sqrt2 = T(0.70710678118654752440);
  T zv;
  if (g < m.mid) {
    zv = X[(m.mid - 1) + (int64_t)g * ldx];
  } else {
    zv = X[m.mid + (int64_t)g * ldx];
    if (e[m.mid - 1] < T(0)) zv = -zv;
  }
  z[g] = zv * inv_sqrt2;
}

// One compare-exchange stage of a batched ascending bitonic sort on (key, index).
template <typename T>
__global__ void dc_bitonic_stage_kernel(T* __restrict__ skey, int* __restrict__ sidx, int64_t total, int np, int k,
                                        int j) {
  const int64_t g = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (g >= total) return;
  const int i = (int)(g & (np - 1));
  const int l = i ^ j;
  if (l <= i) return;
  const int64_t gl = g - i + l;
  const T ki = skey[g], kl = skey[gl];
  const int ii = sidx[g], il = sidx[gl];
  const bool up = ((i & k) == 0);
  const bool i_after_l = (ki > kl) || (ki == kl && ii > il);
  const bool swap = up ? i_after_l : !i_after_l;
  if (swap) {
    skey[g] = kl; skey[gl] = ki;
    sidx[g] = il; sidx[gl] = ii;
  }
}

// Deflation scan (LAPACK laed2 rules).  One workgroup per merge; thread 0 walks the sorted list,
// which the workgroup stages through LDS in chunks.
template <typename T>
__global__ __launch_bounds__(256) void dc_deflate_kernel(int t, int n, int np, T* __restrict__ d,
                                                         const T* __restrict__ e, const T* __restrict__ z,
                                                         const int* __restrict__ sidx, T* __restrict__ dl,
                                                         T* __restrict__ wv, T* __restrict__ dnew,
                                                         int* __restrict__ idx, int* __restrict__ rot_a,
                                                         int* __restrict__ rot_b, T* __restrict__ rot_c,
                                                         T* __restrict__ rot_s, int* __restrict__ kcount,
                                                         int* __restrict__ nrot_out, int* __restrict__ pos1,
                                                         int* __restrict__ pos2, int* __restrict__ sel1,
                                                         int* __restrict__ sel2, int* __restrict__ kc1,
                                                         int* __restrict__ kc2) {
  constexpr int CH = 1024;
  __shared__ T s_d[CH];
  __shared__ T s_z[CH];
  __shared__ int s_p[CH];
  __shared__ T red[256];
  const int q = blockIdx.x;
  const int tid = threadIdx.x;
  const DcMerge m = dc_merge(t, q, n);
  if (m.empty()) {
    if (tid == 0) { kcount[q] = -1; nrot_out[q] = 0; kc1[q] = 0; kc2[q] = 0; }
    return;
  }
  const int lo = m.lo, N = m.hi - m.lo;
  const int n_top = m.mid - m.lo;  // columns [0, n_top) of the block belong to the first child
  const T rho = T(2) * fabs(e[m.mid - 1]);
  T dm = T(0), zm = T(0);
  for (int c = tid; c < N; c += 256) {
    dm = fmax(dm, fabs(d[lo + c]));
    zm = fmax(zm, fabs(z[lo + c]));
  }
  red[tid] = dm;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) { if (tid < s) red[tid] = fmax(red[tid], red[tid + s]); __syncthreads(); }
  dm = red[0];
  __syncthreads();
  red[tid] = zm;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) { if (tid < s) red[tid] = fmax(red[tid], red[tid + s]); __syncthreads(); }
  zm = red[0];
  __syncthreads();
  const T eps = std::numeric_limits<T>::epsilon();
  const T tol = T(8) * eps * fmax(dm, zm);
  if (rho * zm <= tol) {  // nothing couples: the children's eigenpairs are the parent's
    for (int c = tid; c < N; c += 256) { idx[lo + c] = c; dnew[lo + c] = d[lo + c]; }
    if (tid == 0) { kcount[q] = 0; nrot_out[q] = 0; kc1[q] = 0; kc2[q] = 0; }
    return;
  }
  int pj = -1, k = 0, ndefl = 0, nrot = 0;
  int sup_pj = 0, c1 = 0, c2 = 0;  // support of the candidate column: bit 0 top rows, bit 1 bottom rows
  T d_pj = T(0), z_pj = T(0);
  auto keep = [&](int col, T dval, T zval, int sup) {  // a pole of the secular equation
    idx[lo + k] = col; dl[lo + k] = dval; wv[lo + k] = zval;
    pos1[lo + k] = (sup & 1) ? c1 : -1;
    pos2[lo + k] = (sup & 2) ? c2 : -1;
    if (sup & 1) sel1[lo + c1++] = k;
    if (sup & 2) sel2[lo + c2++] = k;
    ++k;
  };
  const int64_t sbase = (int64_t)q * np;
  for (int base = 0; base < N; base += CH) {
    const int cnt = min(CH, N - base);
    __syncthreads();
    for (int c = tid; c < cnt; c += 256) {
      const int li = sidx[sbase + base + c];
      s_p[c] = li;
      s_d[c] = d[lo + li];
      s_z[c] = z[lo + li];
    }
    __syncthreads();
    if (tid == 0) {
      for (int c = 0; c < cnt; ++c) {
        const int nj = s_p[c];
        T dj = s_d[c], zj = s_z[c];
        if (rho * fabs(zj) <= tol) {
          const int slot = N - 1 - ndefl++;
          idx[lo + slot] = nj;
          dnew[lo + slot] = dj;
        } else if (pj < 0) {
          pj = nj; d_pj = dj; z_pj = zj;
          sup_pj = nj < n_top ? 1 : 2;
        } else {
          const int sup_nj = nj < n_top ? 1 : 2;
          T ss = z_pj, cc = zj;
          const T tau = hypot(cc, ss);
          const T tt = dj - d_pj;
          cc /= tau;
          ss = -ss / tau;
          if (fabs(tt * cc * ss) <= tol) {
            zj = tau;
            rot_a[lo + nrot] = pj; rot_b[lo + nrot] = nj;
            rot_c[lo + nrot] = cc; rot_s[lo + nrot] = ss;
            ++nrot;
            const T t2 = d_pj * cc * cc + dj * ss * ss;
            dj = d_pj * ss * ss + dj * cc * cc;
            const int slot = N - 1 - ndefl++;
            idx[lo + slot] = pj;
            dnew[lo + slot] = t2;
            pj = nj; d_pj = dj; z_pj = zj;
            sup_pj |= sup_nj;  // the rotation mixed the two columns
          } else {
            keep(pj, d_pj, z_pj, sup_pj);
            pj = nj; d_pj = dj; z_pj = zj;
            sup_pj = sup_nj;
          }
        }
      }
    }
  }
  if (tid == 0) {
    if (pj >= 0) keep(pj, d_pj, z_pj, sup_pj);
    kcount[q] = k;
    nrot_out[q] = nrot;
    kc1[q] = c1;
    kc2[q] = c2;
  }
}

// Apply the deflation rotations to the columns of the merged block, one thread per row.
template <typename T>
__global__ void dc_rotate_kernel(int t, int n, T* __restrict__ X, int64_t ldx, const int* __restrict__ rot_a,
                                 const int* __restrict__ rot_b, const T* __restrict__ rot_c,
                                 const T* __restrict__ rot_s, const int* __restrict__ nrot) {
  const int q = blockIdx.y;
  const int nr = nrot[q];
  if (nr <= 0) return;
  const DcMerge m = dc_merge(t, q, n);
  const int r = m.lo + blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= m.hi) return;
  for (int i = 0; i < nr; ++i) {
    const int a = rot_a[m.lo + i], b = rot_b[m.lo + i];
    const T c = rot_c[m.lo + i], s = rot_s[m.lo + i];
    T* pa = X + r + (int64_t)(m.lo + a) * ldx;
    T* pb = X + r + (int64_t)(m.lo + b) * ldx;
    const T qa = *pa, qb = *pb;
    *pa = c * qa + s * qb;
    *pb = c * qb - s * qa;
  }
}

// Within the merged block: deflated columns s >= k go to Y[:, s] = X[:, idx[s]]; a surviving column
// s < k goes, for the top rows, to column pos1[s] (if it has support there) and, for the bottom
// rows, to column pos2[s]: the two row ranges of Y hold two differently packed column sets.
template <typename T>
__global__ void dc_gather_kernel(int t, int n, const T* __restrict__ X, int64_t ldx, T* __restrict__ Y, int64_t ldy,
                                 const int* __restrict__ idx, const int* __restrict__ kcount,
                                 const int* __restrict__ pos1, const int* __restrict__ pos2) {
  const int q = blockIdx.z;
  const int k = kcount[q];
  if (k < 0) return;
  const DcMerge m = dc_merge(t, q, n);
  const int r = m.lo + blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= m.hi) return;
  const int N = m.hi - m.lo;
  const int* pos = (r < m.mid) ? pos1 : pos2;
  for (int s = blockIdx.y; s < N; s += gridDim.y) {
    const int dst = (s < k) ? pos[m.lo + s] : s;
    if (dst >= 0) Y[r + (int64_t)(m.lo + dst) * ldy] = X[r + (int64_t)(m.lo + idx[m.lo + s]) * ldx];
  }
}

// Root i of 1 + rho * sum_j w_j^2 / (dl_j - lambda) = 0 on (dl_i, dl_{i+1}).  The unknown is the
// offset mu from the nearer pole, so the differences dl_j - lambda written to `delta` (stride
// dstride) keep full relative accuracy.
template <typename T>
__device__ void dc_secular_root(int i, int k, const T* __restrict__ dl, const T* __restrict__ w, T rho, T* lam_out,
                                T* __restrict__ delta, int64_t dstride) {
  const T eps = std::numeric_limits<T>::epsilon();
  if (k == 1) {
    const T mu = rho * w[0] * w[0];
    *lam_out = dl[0] + mu;
    delta[0] = -mu;
    return;
  }
  const T di = dl[i];
  int org, p1, p2, split;
  T lo, hi;
  if (i < k - 1) {
    const T gap = dl[i + 1] - di;
    const T half = T(0.5) * gap;
    T f = T(1);
    for (int j = 0; j < k; ++j) f += rho * w[j] * w[j] / ((dl[j] - di) - half);
    if (f >= T(0)) { org = i; lo = T(0); hi = half; }
    else { org = i + 1; lo = -half; hi = T(0); }
    p1 = i; p2 = i + 1; split = i;
  } else {
    T s = T(0);
    for (int j = 0; j < k; ++j) s += w[j] * w[j];
    org = k - 1; lo = T(0); hi = rho * s;
    p1 = k - 2; p2 = k - 1; split = k - 2;
  }
  const T dorg = dl[org];
  T mu = T(0.5) * (lo + hi);
  for (int it = 0; it < 120; ++it) {
    if (!(mu > lo && mu < hi)) break;
    T psi = T(0), phi = T(0), dpsi = T(0), dphi = T(0), err = T(1);
    for (int j = 0; j < k; ++j) {
      const T den = (dl[j] - dorg) - mu;
      const T tj = rho * w[j] * w[j] / den;
      const T tt = tj / den;
      if (j <= split) { psi += tj; dpsi += tt; }
      else { phi += tj; dphi += tt; }
      err += fabs(tj);
    }
    const T g = T(1) + psi + phi;
    if (fabs(g) <= T(16) * eps * err) break;
    if (g > T(0)) hi = mu; else lo = mu;
    if (hi - lo <= T(2) * eps * fmax(fabs(lo), fabs(hi))) break;
    const T D1 = (dl[p1] - dorg) - mu, D2 = (dl[p2] - dorg) - mu;
    const T C = g - D1 * dpsi - D2 * dphi;
    const T A = (D1 + D2) * g - D1 * D2 * (dpsi + dphi);
    const T B = D1 * D2 * g;
    T best = mu;
    bool found = false;
    T cand[2];
    int nc = 0;
    if (C == T(0)) {
      if (A != T(0)) cand[nc++] = B / A;
    } else {
      const T disc = A * A - T(4) * B * C;
      if (disc >= T(0)) {
        const T sq = sqrt(disc);
        const T qq = (A >= T(0)) ? A + sq : A - sq;
        cand[nc++] = qq / (T(2) * C);
        if (qq != T(0)) cand[nc++] = T(2) * B / qq;
      }
    }
    for (int c = 0; c < nc; ++c) {
      const T x = mu + cand[c];
      if (x > lo && x < hi && (!found || fabs(cand[c]) < fabs(best - mu))) { best = x; found = true; }
    }
    if (!found) {
      if (lo > T(0) && hi > T(16) * lo) best = sqrt(lo) * sqrt(hi);
      else if (hi < T(0) && lo < T(16) * hi) best = -(sqrt(-lo) * sqrt(-hi));
      else best = T(0.5) * (lo + hi);
      if (!(best > lo && best < hi)) break;
    }
    mu = best;
  }
  if (!(mu > lo && mu < hi)) mu = T(0.5) * (lo + hi);
  *lam_out = dorg + mu;
  for (int j = 0; j < k; ++j) delta[(int64_t)j * dstride] = (dl[j] - dorg) - mu;
}

// The same iteration with the sums over the poles spread over the 64 lanes of a wavefront (lane l
// takes poles l, l + 64, ...; xor-butterfly sums give every lane the same total), for merges with
// many poles, where a thread per root leaves most of the chip idle.  Writes the root, its origin
// pole and its offset; dc_delta_kernel then forms the differences with lanes along the roots.
template <typename T>
__device__ __forceinline__ T dc_wave_sum(T v) {
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) v += __shfl_xor(v, m, 64);
  return v;
}

template <typename T>
__device__ void dc_secular_root_wave(int i, int k, int lane, const T* __restrict__ dl, const T* __restrict__ w, T rho,
                                     T* lam_out, T* mu_out, int* org_out) {
  const T eps = std::numeric_limits<T>::epsilon();
  if (k == 1) {
    const T mu = rho * w[0] * w[0];
    if (lane == 0) { *lam_out = dl[0] + mu; *mu_out = mu; *org_out = 0; }
    return;
  }
  const T di = dl[i];
  int org, p1, p2, split;
  T lo, hi;
  if (i < k - 1) {
    const T gap = dl[i + 1] - di;
    const T half = T(0.5) * gap;
    T f = T(0);
    for (int j = lane; j < k; j += 64) f += rho * w[j] * w[j] / ((dl[j] - di) - half);
    f = T(1) + dc_wave_sum(f);
    if (f >= T(0)) { org = i; lo = T(0); hi = half; }
    else { org = i + 1; lo = -half; hi = T(0); }
    p1 = i; p2 = i + 1; split = i;
  } else {
    T s = T(0);
    for (int j = lane; j < k; j += 64) s += w[j] * w[j];
    s = dc_wave_sum(s);
    org = k - 1; lo = T(0); hi = rho * s;
    p1 = k - 2; p2 = k - 1; split = k - 2;
  }
  const T dorg = dl[org];
  T mu = T(0.5) * (lo + hi);
  for (int it = 0; it < 120; ++it) {
    if (!(mu > lo && mu < hi)) break;
    T psi = T(0), phi = T(0), dpsi = T(0), dphi = T(0), err = T(0);
    for (int j = lane; j < k; j += 64) {
      const T den = (dl[j] - dorg) - mu;
      const T tj = rho * w[j] * w[j] / den;
      const T tt = tj / den;
      if (j <= split) { psi += tj; dpsi += tt; }
      else { phi += tj; dphi += tt; }
      err += fabs(tj);
    }
    psi = dc_wave_sum(psi); phi = dc_wave_sum(phi); dpsi = dc_wave_sum(dpsi); dphi = dc_wave_sum(dphi);
    err = T(1) + dc_wave_sum(err);
    const T g = T(1) + psi + phi;
    if (fabs(g) <= T(16) * eps * err) break;
    if (g > T(0)) hi = mu; else lo = mu;
    if (hi - lo <= T(2) * eps * fmax(fabs(lo), fabs(hi))) break;
    const T D1 = (dl[p1] - dorg) - mu, D2 = (dl[p2] - dorg) - mu;
    const T C = g - D1 * dpsi - D2 * dphi;
    const T A = (D1 + D2) * g - D1 * D2 * (dpsi + dphi);
    const T B = D1 * D2 * g;
    T best = mu;
    bool found = false;
    T cand[2];
    int nc = 0;
    if (C == T(0)) {
      if (A != T(0)) cand[nc++] = B / A;
    } else {
      const T disc = A * A - T(4) * B * C;
      if (disc >= T(0)) {
        const T sq = sqrt(disc);
        const T qq = (A >= T(0)) ? A + sq : A - sq;
        cand[nc++] = qq / (T(2) * C);
        if (qq != T(0)) cand[nc++] = T(2) * B / qq;
      }
    }
    for (int c = 0; c < nc; ++c) {
      const T x = mu + cand[c];
      if (x > lo && x < hi && (!found || fabs(cand[c]) < fabs(best - mu))) { best = x; found = true; }
    }
    if (!found) {
      if (lo > T(0) && hi > T(16) * lo) best = sqrt(lo) * sqrt(hi);
      else if (hi < T(0) && lo < T(16) * hi) best = -(sqrt(-lo) * sqrt(-hi));
      else best = T(0.5) * (lo + hi);
      if (!(best > lo && best < hi)) break;
    }
    mu = best;
  }
  if (!(mu > lo && mu < hi)) mu = T(0.5) * (lo + hi);
  if (lane == 0) { *lam_out = dorg + mu; *mu_out = mu; *org_out = org; }
}

template <typename T>
__global__ __launch_bounds__(256) void dc_secular_wave_kernel(int t, int n, const T* __restrict__ e,
                                                              const T* __restrict__ dl, const T* __restrict__ wv,
                                                              const int* __restrict__ kcount, T* __restrict__ dnew,
                                                              T* __restrict__ mu, int* __restrict__ org) {
  const int q = blockIdx.y;
  const int k = kcount[q];
  const int i = blockIdx.x * 4 + (threadIdx.x >> 6);  // one wavefront per root
  if (i >= k) return;
  const DcMerge m = dc_merge(t, q, n);
  const T rho = T(2) * fabs(e[m.mid - 1]);
  dc_secular_root_wave<T>(i, k, threadIdx.x & 63, dl + m.lo, wv + m.lo, rho, dnew + m.lo + i, mu + m.lo + i,
                          org + m.lo + i);
}

// deltaT[i, j] = (dl_j - dl_org(i)) - mu_i at S[(lo + i) + (lo + j) * lds]: lanes along the roots.
template <typename T>
__global__ __launch_bounds__(256) void dc_delta_kernel(int t, int n, const T* __restrict__ dl,
                                                       const int* __restrict__ kcount, const T* __restrict__ mu,
                                                       const int* __restrict__ org, T* __restrict__ S, int64_t lds) {
  const int q = blockIdx.z;
  const int k = kcount[q];
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= k) return;
  const int lo = dc_bound(t, q, n);
  const T dorg = dl[lo + org[lo + i]], m = mu[lo + i];
  T* row = S + (lo + i) + (int64_t)lo * lds;
  for (int j = blockIdx.y; j < k; j += gridDim.y) row[(int64_t)j * lds] = (dl[lo + j] - dorg) - m;
}

template <typename T>
__global__ __launch_bounds__(64) void dc_secular_kernel(int t, int n, const T* __restrict__ e,
                                                        const T* __restrict__ dl, const T* __restrict__ wv,
                                                        const int* __restrict__ kcount, T* __restrict__ dnew,
                                                        T* __restrict__ S, int64_t lds) {
  const int q = blockIdx.y;
  const int k = kcount[q];
  const int i = blockIdx.x * 64 + threadIdx.x;
  if (i >= k) return;
  const DcMerge m = dc_merge(t, q, n);
  const T rho = T(2) * fabs(e[m.mid - 1]);
  // deltaT[i, j] lives at S[(lo + i) + (lo + j) * lds]: lanes (roots) are contiguous
  dc_secular_root<T>(i, k, dl + m.lo, wv + m.lo, rho, dnew + m.lo + i, S + (m.lo + i) + (int64_t)m.lo * lds, lds);
}

// zhat_j = sign(w_j) sqrt( -deltaT[j,j] * prod_{i != j} deltaT[i,j] / (dl_j - dl_i) ).
template <typename T>
__global__ __launch_bounds__(256) void dc_zhat_kernel(int t, int n, const T* __restrict__ dl, const T* __restrict__ wv,
                                                      const int* __restrict__ kcount, const T* __restrict__ S,
                                                      int64_t lds, T* __restrict__ zhat) {
  __shared__ T red[256];
  const int q = blockIdx.y;
  const int k = kcount[q];
  const int j = blockIdx.x;
  if (j >= k) return;
  const int lo = dc_bound(t, q, n);
  const T dj = dl[lo + j];
  const T* col = S + lo + (int64_t)(lo + j) * lds;
  T prod = T(1);
  for (int i = threadIdx.x; i < k; i += 256) {
    const T dt = col[i];
    prod *= (i == j) ? dt : dt / (dj - dl[lo + i]);
  }
  red[threadIdx.x] = prod;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if (threadIdx.x < s) red[threadIdx.x] *= red[threadIdx.x + s];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    const T v = sqrt(fmax(-red[0], T(0)));
    zhat[lo + j] = (wv[lo + j] < T(0)) ? -v : v;
  }
}

// Column i of the rank-one eigenvector matrix, u_i[j] = zhat_j / deltaT[i, j] normalised, stored
// transposed in place of deltaT.  Two passes over a 2-D grid (roots x kDcNormChunks slices of the
// poles): partial squared norms, then every thread sums the partials of its root in slice order
// and writes its slice.
constexpr int kDcNormChunks = 32;

template <typename T>
__global__ void dc_form_u_norm_kernel(int t, int n, const int* __restrict__ kcount, const T* __restrict__ zhat,
                                      const T* __restrict__ S, int64_t lds, T* __restrict__ norm_part) {
  const int q = blockIdx.z;
  const int k = kcount[q];
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= k) return;
  const int lo = dc_bound(t, q, n);
  const int chunk = (k + kDcNormChunks - 1) / kDcNormChunks;
  const int j0 = blockIdx.y * chunk, j1 = min(k, j0 + chunk);
  const T* row = S + (lo + i) + (int64_t)lo * lds;
  T nrm2 = T(0);
  for (int j = j0; j < j1; ++j) {
    const T s = zhat[lo + j] / row[(int64_t)j * lds];
    nrm2 += s * s;
  }
  norm_part[(int64_t)blockIdx.y * n + lo + i] = nrm2;
}

template <typename T>
__global__ void dc_form_u_kernel(int t, int n, const int* __restrict__ kcount, const T* __restrict__ zhat,
                                 T* __restrict__ S, int64_t lds, const T* __restrict__ norm_part) {
  const int q = blockIdx.z;
  const int k = kcount[q];
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= k) return;
  const int lo = dc_bound(t, q, n);
  const int chunk = (k + kDcNormChunks - 1) / kDcNormChunks;
  const int j0 = blockIdx.y * chunk, j1 = min(k, j0 + chunk);
  T nrm2 = T(0);
  for (int c = 0; c < kDcNormChunks; ++c) nrm2 += norm_part[(int64_t)c * n + lo + i];
  const T inv = T(1) / sqrt(nrm2);
  T* row = S + (lo + i) + (int64_t)lo * lds;
  for (int j = j0; j < j1; ++j) row[(int64_t)j * lds] = zhat[lo + j] / row[(int64_t)j * lds] * inv;
}

template <typename T>
__global__ void dc_setup_gemm_kernel(int t, int n, int nq, const int* __restrict__ kcount, const int* __restrict__ kc1,
                                     const int* __restrict__ kc2, const int* __restrict__ sel1,
                                     const int* __restrict__ sel2, const T* __restrict__ Y, int64_t ldy,
                                     const T* __restrict__ S, int64_t lds, T* __restrict__ X, int64_t ldx,
                                     BatchedGemm<T>* __restrict__ batch) {
  using Cfg = typename DefaultTile<T>::type;
  const int q = blockIdx.x * blockDim.x + threadIdx.x;
  if (q >= nq) return;
  const int k = kcount[q];
  BatchedGemm<T> b;
  if (k <= 0) {
    b.p.M = 0; b.p.N = 0; b.p.K = 0; b.p.num_tiles = 0;
    batch[2 * q] = b;
    batch[2 * q + 1] = b;
    return;
  }
  const DcMerge m = dc_merge(t, q, n);
  const int64_t o = m.lo;
  // X[rows, 0:k] = Y[rows, 0:k_half] * U[sel, :] with U[j, i] = S[i + j*lds] (stored transposed), once
  // for the top rows with the top-supported poles and once for the bottom rows
  fill_batched<T, Cfg>(b, 0, 1, m.mid - m.lo, k, kc1[q], Y + o + o * ldy, ldy, S + o + o * lds, lds, X + o + o * ldx, ldx,
                       T(1), T(0));
  b.p.ksel_b = sel1 + m.lo;
  batch[2 * q] = b;
  fill_batched<T, Cfg>(b, 0, 1, m.hi - m.mid, k, kc2[q], Y + m.mid + o * ldy, ldy, S + o + o * lds, lds,
                       X + m.mid + o * ldx, ldx, T(1), T(0));
  b.p.ksel_b = sel2 + m.lo;
  batch[2 * q + 1] = b;
}

// Deflated columns pass through unchanged; d takes the merged eigenvalues.
template <typename T>
__global__ void dc_finish_kernel(int t, int n, const int* __restrict__ kcount, const T* __restrict__ Y, int64_t ldy,
                                 T* __restrict__ X, int64_t ldx, const T* __restrict__ dnew, T* __restrict__ d) {
  const int q = blockIdx.z;
  const int k = kcount[q];
  if (k < 0) return;
  const DcMerge m = dc_merge(t, q, n);
  const int N = m.hi - m.lo;
  const int rl = blockIdx.x * blockDim.x + threadIdx.x;
  if (blockIdx.y == 0 && rl < N) d[m.lo + rl] = dnew[m.lo + rl];
  const int r = m.lo + rl;
  if (r >= m.hi) return;
  for (int s = k + blockIdx.y; s < N; s += gridDim.y) X[r + (int64_t)(m.lo + s) * ldx] = Y[r + (int64_t)(m.lo + s) * ldy];
}

// w_out[s] = scale * d[order[s]];  Z[:, s] = X[:, order[s]].
template <typename T>
__global__ void dc_output_kernel(int n, const T* __restrict__ d, const int* __restrict__ order,
                                 const T* __restrict__ scal, T* __restrict__ w_out, const T* __restrict__ X,
                                 int64_t ldx, T* __restrict__ Z, int64_t ldz) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= n) return;
  if (blockIdx.y == 0) w_out[r] = scal[0] * d[order[r]];
  for (int s = blockIdx.y; s < n; s += gridDim.y) Z[r + (int64_t)s * ldz] = X[r + (int64_t)order[s] * ldx];
}

template <typename T>
__global__ void dc_final_keys_kernel(int n, int np, const T* __restrict__ d, T* __restrict__ skey,
                                     int* __restrict__ sidx) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= np) return;
  sidx[c] = c;
  skey[c] = (c < n) ? d[c] : std::numeric_limits<T>::infinity();
}

static inline int dc_next_pow2(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

template <typename T>
static inline void dc_batched_sort(hipStream_t s, const DcWorkspace<T>& ws, int np, int nq) {
  const int64_t total = (int64_t)np * nq;
  const unsigned blocks = (unsigned)ceil_div64(total, 256);
  for (int k = 2; k <= np; k <<= 1)
    for (int j = k >> 1; j > 0; j >>= 1)
      hipLaunchKernelGGL((dc_bitonic_stage_kernel<T>), dim3(blocks), dim3(256), 0, s, ws.skey, ws.sidx, total, np, k, j);
}

// Eigen-decomposition of the tridiagonal (d0, e0): ascending eigenvalues into w_out, matching
// eigenvectors into the columns of Z.  Y is an n x n scratch matrix (may be Z itself).
template <typename T>
static inline int stedc(hipStream_t s, int n, const T* d0, const T* e0, T* w_out, T* Z, int64_t ldz,
                        const DcWorkspace<T>& ws) {
  using Cfg = typename DefaultTile<T>::type;
  T* Y = Z;
  const int64_t ldy = ldz;
  hipLaunchKernelGGL((dc_scale_kernel<T>), dim3(1), dim3(1024), 0, s, d0, e0, n, ws.scal);
  hipLaunchKernelGGL((dc_init_kernel<T>), dim3((unsigned)ceil_div64(n, 256)), dim3(256), 0, s, d0, e0, n, ws.scal, ws.d,
                     ws.e);
  const unsigned rb = (unsigned)ceil_div64(n, 256);
  hipLaunchKernelGGL((set_identity_kernel<T>), dim3(rb, (unsigned)std::min(n, 4096)), dim3(256), 0, s, ws.X, ws.ldx, n);
  SOAPMI_LAUNCH_CHECK();
  int depth = 0;
  while ((1 << depth) < n) ++depth;
  for (int t = depth - 1; t >= 0; --t) {
    const int nq = 1 << t;
    const int nmax = (int)ceil_div64(n, nq);
    const int np = dc_next_pow2(nmax);
    const unsigned rbl = (unsigned)ceil_div64(nmax, 256);
    const unsigned ycols = (unsigned)std::min(nmax, 2048);
    hipLaunchKernelGGL((dc_z_keys_kernel<T>), dim3((unsigned)ceil_div64(np, 256), nq), dim3(256), 0, s, t, n, np, ws.X,
                       ws.ldx, ws.d, ws.e, ws.z, ws.skey, ws.sidx);
    dc_batched_sort<T>(s, ws, np, nq);
    hipLaunchKernelGGL((dc_deflate_kernel<T>), dim3(nq), dim3(256), 0, s, t, n, np, ws.d, ws.e, ws.z, ws.sidx, ws.dl,
                       ws.wv, ws.dnew, ws.idx, ws.rot_a, ws.rot_b, ws.rot_c, ws.rot_s, ws.kcount, ws.nrot, ws.pos1, ws.pos2,
                       ws.sel1, ws.sel2, ws.kc1, ws.kc2);
    hipLaunchKernelGGL((dc_rotate_kernel<T>), dim3(rbl, nq), dim3(256), 0, s, t, n, ws.X, ws.ldx, ws.rot_a, ws.rot_b,
                       ws.rot_c, ws.rot_s, ws.nrot);
    hipLaunchKernelGGL((dc_gather_kernel<T>), dim3(rbl, ycols, nq), dim3(256), 0, s, t, n, ws.X, ws.ldx, Y, ldy, ws.idx,
                       ws.kcount, ws.pos1, ws.pos2);
    if (nmax >= 256) {
      hipLaunchKernelGGL((dc_secular_wave_kernel<T>), dim3((unsigned)ceil_div64(nmax, 4), nq), dim3(256), 0, s, t, n,
                         ws.e, ws.dl, ws.wv, ws.kcount, ws.dnew, ws.mu, ws.org);
      hipLaunchKernelGGL((dc_delta_kernel<T>), dim3(rbl, ycols, nq), dim3(256), 0, s, t, n, ws.dl, ws.kcount, ws.mu,
                         ws.org, ws.S, ws.lds);
    } else {
      hipLaunchKernelGGL((dc_secular_kernel<T>), dim3((unsigned)ceil_div64(nmax, 64), nq), dim3(64), 0, s, t, n, ws.e,
                         ws.dl, ws.wv, ws.kcount, ws.dnew, ws.S, ws.lds);
    }
    hipLaunchKernelGGL((dc_zhat_kernel<T>), dim3(nmax, nq), dim3(256), 0, s, t, n, ws.dl, ws.wv, ws.kcount, ws.S, ws.lds,
                       ws.zhat);
    hipLaunchKernelGGL((dc_form_u_norm_kernel<T>), dim3(rbl, kDcNormChunks, nq), dim3(256), 0, s, t, n, ws.kcount, ws.zhat,
                       ws.S, ws.lds, ws.norm_part);
    hipLaunchKernelGGL((dc_form_u_kernel<T>), dim3(rbl, kDcNormChunks, nq), dim3(256), 0, s, t, n, ws.kcount, ws.zhat,
                       ws.S, ws.lds, ws.norm_part);
    hipLaunchKernelGGL((dc_setup_gemm_kernel<T>), dim3((unsigned)ceil_div64(nq, 256)), dim3(256), 0, s, t, n, nq,
                       ws.kcount, ws.kc1, ws.kc2, ws.sel1, ws.sel2, Y, ldy, ws.S, ws.lds, ws.X, ws.ldx, ws.batch);
    const int half = nmax / 2 + 1;  // a child has at most this many rows
    const int tiles = (int)(ceil_div64(half, Cfg::BM) * ceil_div64(nmax, Cfg::BN));
    hipLaunchKernelGGL((gemm_batched_kernel<T, Cfg>), dim3(8 * (unsigned)ceil_div64(tiles, 8), 1, 2 * nq), dim3(Cfg::NT),
                       0, s, ws.batch);
    hipLaunchKernelGGL((dc_finish_kernel<T>), dim3(rbl, ycols, nq), dim3(256), 0, s, t, n, ws.kcount, Y, ldy, ws.X,
                       ws.ldx, ws.dnew, ws.d);
    SOAPMI_LAUNCH_CHECK();
  }
  // final ordering
  const int np = dc_next_pow2(n);
  hipLaunchKernelGGL((dc_final_keys_kernel<T>), dim3((unsigned)ceil_div64(np, 256)), dim3(256), 0, s, n, np, ws.d,
                     ws.skey, ws.sidx);
  dc_batched_sort<T>(s, ws, np, 1);
  hipLaunchKernelGGL((dc_output_kernel<T>), dim3(rb, (unsigned)std::min(n, 2048)), dim3(256), 0, s, n, ws.d, ws.sidx,
                     ws.scal, w_out, ws.X, ws.ldx, Z, ldz);
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

}  // namespace soapmi
