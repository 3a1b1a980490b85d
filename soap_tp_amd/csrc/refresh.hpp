// Kernels of the basis refresh other than the products and the QR: column dots (eigenvalue
// estimates), descending argsort, row/column gathers.
#pragma once
#include "common.hpp"

namespace soapmi {

// est[j] = sum_i Q[i, j] * W[i, j]   (factorizations.py:255-257).  One wavefront per column (four
// columns per workgroup); a lane takes every 64th group of four rows with 16-byte loads when the
// columns are aligned for them, and the wavefront's partial sums meet in a fixed xor-butterfly: the
// estimates, and hence the sort order, are reproducible.
template <typename T>
__global__ __launch_bounds__(256) void coldot_kernel(const T* __restrict__ Q, int64_t ldq, const T* __restrict__ W,
                                                     int64_t ldw, int n_rows, int n_cols, T* __restrict__ est,
                                                     int vectors) {
  const int lane = threadIdx.x & 63;
  const int j = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (j >= n_cols) return;
  const T* q = Q + (int64_t)j * ldq;
  const T* w = W + (int64_t)j * ldw;
  T s = T(0);
  if (vectors) {
    using V = typename Vec16<T>::type;
    constexpr int VW = Vec16<T>::W;
    for (int i = lane * VW; i < n_rows; i += 64 * VW) {
      const V a = *reinterpret_cast<const V*>(q + i);
      const V b = *reinterpret_cast<const V*>(w + i);
      const T* pa = reinterpret_cast<const T*>(&a);
      const T* pb = reinterpret_cast<const T*>(&b);
#pragma unroll
      for (int e = 0; e < VW; ++e) s += pa[e] * pb[e];
    }
  } else {
    for (int i = lane; i < n_rows; i += 64) s += q[i] * w[i];
  }
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) s += __shfl_xor(s, m, 64);
  if (lane == 0) est[j] = s;
}

// Total order used by the argsort: NaN first (torch.argsort(descending=True) treats NaN as the
// largest value), then larger value first, ties by smaller index (torch leaves the order of ties
// unspecified: factorizations.py:271).
__device__ __forceinline__ bool sorts_before(float va, int ia, float vb, int ib) {
  const bool na = va != va, nb = vb != vb;
  if (na || nb) return (na && !nb) || (na == nb && ia < ib);
  if (va > vb) return true;
  if (va < vb) return false;
  return ia < ib;
}

// Argsort by counting, for up to kArgsortRankMax keys: every workgroup holds all keys in LDS (mapped
// to unsigned integers that order like sorts_before: NaN first, larger value first, -0 = +0) and each
// key's four threads count the keys that sort before it; that count is the key's position.  n^2 integer
// comparisons spread over 4n threads, no exchanges and no atomics: about a tenth of the time of a
// bitonic network run by one workgroup at n = 11008.
constexpr int kArgsortRankMax = 16384;

__device__ __forceinline__ unsigned argsort_key(float v) {
  if (v != v) return 0xffffffffu;
  unsigned u = __float_as_uint(v);
  if (u == 0x80000000u) u = 0u;  // -0 ties with +0
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__global__ __launch_bounds__(256) void argsort_desc_rank_kernel(const float* __restrict__ keys, int n,
                                                                int64_t* __restrict__ order) {
  extern __shared__ __attribute__((aligned(16))) unsigned s_key[];  // (n rounded up to 4) keys
  const int n4 = (n + 3) & ~3;
  for (int j = threadIdx.x; j < n4; j += 256) s_key[j] = (j < n) ? argsort_key(keys[j]) : 0u;
  __syncthreads();
  // four neighbouring lanes share a key and take a quarter of the comparisons each
  const int i = blockIdx.x * 64 + (threadIdx.x >> 2), part = threadIdx.x & 3;
  const int quarter = ((n4 / 4) + 3) & ~3;
  const int j0 = min(n4, part * quarter), j1 = min(n4, j0 + quarter);
  const unsigned mine = s_key[min(i, n - 1)];
  int before = 0;
  for (int j = j0; j < j1; j += 4) {
    const uint4 k4 = *reinterpret_cast<const uint4*>(s_key + j);
    const unsigned kk[4] = {k4.x, k4.y, k4.z, k4.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int jj = j + e;
      // padding entries (jj >= n) carry key 0, below every real key (-inf maps to 0x007fffff), and an
      // index above every real one: never before a real key
      before += (kk[e] > mine || (kk[e] == mine && jj < i)) ? 1 : 0;
    }
  }
  before += __shfl_xor(before, 1, 64);
  before += __shfl_xor(before, 2, 64);
  if (part == 0 && i < n) order[before] = (int64_t)i;
}

// Global-memory bitonic stage for key counts that do not fit LDS.
__global__ void argsort_init_kernel(const float* __restrict__ keys, int n, int np2, float* v, int* id) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= np2) return;
  v[i] = (i < n) ? keys[i] : __int_as_float(0xff800000);  // padding: -inf with an index above every real one
  id[i] = i;
}
__global__ void argsort_stage_kernel(float* v, int* id, int np2, int k, int j) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= np2) return;
  const int l = i ^ j;
  if (l > i) {
    const bool up = ((i & k) == 0);
    const float vi = v[i], vl = v[l];
    const int ii = id[i], il = id[l];
    const bool swap = up ? sorts_before(vl, il, vi, ii) : sorts_before(vi, ii, vl, il);
    if (swap) {
      v[i] = vl; v[l] = vi;
      id[i] = il; id[l] = ii;
    }
  }
}
__global__ void argsort_finish_kernel(const int* id, int n, int64_t* order) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) order[i] = (int64_t)id[i];
}

// out[i, j] = in[row_order[i], col_order[j]]  (optimizer.py:408 semantics); a null order is the
// identity.  Three kernels, chosen by launch_gather2d:
//   gather2d_columns_kernel  rows not permuted, everything 16-byte aligned: a thread moves four
//                            consecutive rows of a column per load, eight columns per thread
//   gather2d_lds_kernel      rows permuted, a source column fits in LDS (up to 16384 rows): a workgroup
//                            reads two source columns (one above 8192 rows) with coalesced loads, then
//                            serves its output rows from LDS, so the matrix crosses HBM once each way
//                            however scattered the row order is
//   gather2d_kernel          anything else (lanes along i: coalesced when rows are not permuted)
template <typename T>
__global__ void gather2d_kernel(const T* __restrict__ in, int64_t ldi, T* __restrict__ out, int64_t ldo, int rows,
                                int cols, const int64_t* __restrict__ row_order,
                                const int64_t* __restrict__ col_order) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows) return;
  const int64_t si = row_order ? row_order[i] : (int64_t)i;
  for (int j = blockIdx.y; j < cols; j += gridDim.y) {
    const int64_t sj = col_order ? col_order[j] : (int64_t)j;
    out[i + (int64_t)j * ldo] = in[si + sj * ldi];
  }
}

constexpr int kGatherColsPerThread = 8;

__global__ __launch_bounds__(256) void gather2d_columns_kernel(const float* __restrict__ in, int64_t ldi,
                                                               float* __restrict__ out, int64_t ldo, int rows, int cols,
                                                               const int64_t* __restrict__ col_order) {
  const int i4 = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i4 >= rows) return;
  const int j0 = blockIdx.y * kGatherColsPerThread;
  float4 v[kGatherColsPerThread];
#pragma unroll
  for (int c = 0; c < kGatherColsPerThread; ++c) {
    const int j = min(j0 + c, cols - 1);
    const int64_t sj = col_order ? col_order[j] : (int64_t)j;
    v[c] = *reinterpret_cast<const float4*>(in + i4 + sj * ldi);
  }
#pragma unroll
  for (int c = 0; c < kGatherColsPerThread; ++c)
    if (j0 + c < cols) *reinterpret_cast<float4*>(out + i4 + (int64_t)(j0 + c) * ldo) = v[c];
}

// LDS holds COLS source columns of up to kGatherLdsFloats / COLS rows each (64 KB in all): two
// columns per workgroup up to 8192 rows, one column up to 16384 rows.  With VEC every global access
// moves 16 bytes: the source columns are read as float4, and a thread produces four consecutive
// output rows per store (their four source rows come out of LDS one by one).
constexpr int kGatherLdsFloats = 16384;

template <int COLS, bool VEC>
__global__ __launch_bounds__(256) void gather2d_lds_kernel(const float* __restrict__ in, int64_t ldi,
                                                           float* __restrict__ out, int64_t ldo, int rows, int cols,
                                                           const int64_t* __restrict__ row_order,
                                                           const int64_t* __restrict__ col_order) {
  constexpr int CAP = kGatherLdsFloats / COLS;
  __shared__ __attribute__((aligned(16))) float column[COLS][CAP];
  const int j0 = COLS * blockIdx.x;
  int64_t src[COLS];
#pragma unroll
  for (int c = 0; c < COLS; ++c) {
    const int j = min(j0 + c, cols - 1);
    src[c] = col_order ? col_order[j] : (int64_t)j;
  }
  if (VEC) {
    for (int i4 = threadIdx.x * 4; i4 < rows; i4 += 1024) {
#pragma unroll
      for (int c = 0; c < COLS; ++c)
        *reinterpret_cast<float4*>(&column[c][i4]) = *reinterpret_cast<const float4*>(in + i4 + src[c] * ldi);
    }
  } else {
    for (int i = threadIdx.x; i < rows; i += 256) {
#pragma unroll
      for (int c = 0; c < COLS; ++c) column[c][i] = in[i + src[c] * ldi];
    }
  }
  __syncthreads();
  if (VEC) {
    for (int i4 = threadIdx.x * 4; i4 < rows; i4 += 1024) {
      const longlong2 a = *reinterpret_cast<const longlong2*>(row_order + i4);
      const longlong2 b = *reinterpret_cast<const longlong2*>(row_order + i4 + 2);
      const int s0 = (int)a.x, s1 = (int)a.y, s2 = (int)b.x, s3 = (int)b.y;
#pragma unroll
      for (int c = 0; c < COLS; ++c) {
        if (j0 + c < cols) {
          const float4 v = make_float4(column[c][s0], column[c][s1], column[c][s2], column[c][s3]);
          *reinterpret_cast<float4*>(out + i4 + (int64_t)(j0 + c) * ldo) = v;
        }
      }
    }
  } else {
    for (int i = threadIdx.x; i < rows; i += 256) {
      const int si = (int)row_order[i];
#pragma unroll
      for (int c = 0; c < COLS; ++c)
        if (j0 + c < cols) out[i + (int64_t)(j0 + c) * ldo] = column[c][si];
    }
  }
}

static inline bool aligned16_columns(const void* p, int64_t ld, int64_t rows) {
  return reinterpret_cast<uintptr_t>(p) % 16 == 0 && ld % 4 == 0 && rows % 4 == 0;
}

// out = in[row_order][:, col_order] (null orders: identity) with the kernel that fits.
static inline void launch_gather2d(hipStream_t s, const float* in, int64_t ldi, float* out, int64_t ldo, int64_t rows,
                                   int64_t cols, const int64_t* row_order, const int64_t* col_order) {
  if (rows <= 0 || cols <= 0) return;
  if (!row_order && aligned16_columns(in, ldi, rows) && aligned16_columns(out, ldo, rows)) {
    const dim3 grid((unsigned)ceil_div64(rows, 1024), (unsigned)ceil_div64(cols, kGatherColsPerThread));
    hipLaunchKernelGGL(gather2d_columns_kernel, grid, dim3(256), 0, s, in, ldi, out, ldo, (int)rows, (int)cols, col_order);
  } else if (row_order && rows <= kGatherLdsFloats) {
    // (row_order comes from an int64 allocation: 16-byte aligned whenever the data pointers are)
    const bool vec = aligned16_columns(in, ldi, rows) && aligned16_columns(out, ldo, rows) &&
                     reinterpret_cast<uintptr_t>(row_order) % 16 == 0;
    const dim3 two((unsigned)ceil_div64(cols, 2)), one((unsigned)cols);
    if (rows <= kGatherLdsFloats / 2) {
      if (vec) hipLaunchKernelGGL((gather2d_lds_kernel<2, true>), two, dim3(256), 0, s, in, ldi, out, ldo, (int)rows,
                                  (int)cols, row_order, col_order);
      else hipLaunchKernelGGL((gather2d_lds_kernel<2, false>), two, dim3(256), 0, s, in, ldi, out, ldo, (int)rows,
                              (int)cols, row_order, col_order);
    } else {
      if (vec) hipLaunchKernelGGL((gather2d_lds_kernel<1, true>), one, dim3(256), 0, s, in, ldi, out, ldo, (int)rows,
                                  (int)cols, row_order, col_order);
      else hipLaunchKernelGGL((gather2d_lds_kernel<1, false>), one, dim3(256), 0, s, in, ldi, out, ldo, (int)rows,
                              (int)cols, row_order, col_order);
    }
  } else {
    const dim3 grid((unsigned)ceil_div64(rows, 256), (unsigned)(cols < 8192 ? cols : 8192));
    hipLaunchKernelGGL((gather2d_kernel<float>), grid, dim3(256), 0, s, in, ldi, out, ldo, (int)rows, (int)cols,
                       row_order, col_order);
  }
}

// flags[0] = 1 unless `order` is a permutation of range(n).  `seen` must be zeroed (n ints).
__global__ void check_permutation_kernel(const int64_t* __restrict__ order, int n, int* seen, int* flags) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int64_t v = order[i];
  if (v < 0 || v >= n) {
    flags[0] = 1;
    return;
  }
  if (atomicAdd(&seen[v], 1) != 0) flags[0] = 1;
}

}  // namespace soapmi
