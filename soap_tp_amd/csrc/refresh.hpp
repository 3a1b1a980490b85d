// Kernels of the basis refresh other than the products and the QR: column dots (eigenvalue
// estimates), descending argsort, row/column gathers.
#pragma once
#include "common.hpp"

namespace soapmi {

// est[j] = sum_i Q[i, j] * W[i, j]   (factorizations.py:255-257).  One workgroup per column,
// fixed reduction tree, so the estimates (and hence the sort order) are reproducible.
template <typename T>
__global__ void coldot_kernel(const T* __restrict__ Q, int64_t ldq, const T* __restrict__ W, int64_t ldw, int n_rows,
                              T* __restrict__ est) {
  __shared__ T red[256];
  const int j = blockIdx.x;
  T s = T(0);
  for (int i = threadIdx.x; i < n_rows; i += 256) s += Q[i + (int64_t)j * ldq] * W[i + (int64_t)j * ldw];
  red[threadIdx.x] = s;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if (threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) est[j] = red[0];
}

// Total order used by the argsort: larger value first, ties by smaller index, NaN last.
// (torch.argsort(descending=True) leaves the order of ties unspecified: factorizations.py:271.)
__device__ __forceinline__ bool sorts_before(float va, int ia, float vb, int ib) {
  const bool na = va != va, nb = vb != vb;
  if (na || nb) return (!na && nb) || (na == nb && ia < ib);
  if (va > vb) return true;
  if (va < vb) return false;
  return ia < ib;
}

// Bitonic argsort of up to `np2` (power of two) keys entirely in LDS: one workgroup.
__global__ void argsort_desc_lds_kernel(const float* __restrict__ keys, int n, int np2, int64_t* __restrict__ order) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float* v = reinterpret_cast<float*>(smem);
  int* id = reinterpret_cast<int*>(smem + sizeof(float) * (size_t)np2);
  const int tid = threadIdx.x, nt = blockDim.x;
  for (int i = tid; i < np2; i += nt) {
    v[i] = (i < n) ? keys[i] : __int_as_float(0x7fc00000);  // padding sorts last (NaN, large index)
    id[i] = i;
  }
  __syncthreads();
  for (int k = 2; k <= np2; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int i = tid; i < np2; i += nt) {
        const int l = i ^ j;
        if (l > i) {
          const bool up = ((i & k) == 0);  // ascending position = "sorts_before" order
          const float vi = v[i], vl = v[l];
          const int ii = id[i], il = id[l];
          const bool swap = up ? sorts_before(vl, il, vi, ii) : sorts_before(vi, ii, vl, il);
          if (swap) {
            v[i] = vl; v[l] = vi;
            id[i] = il; id[l] = ii;
          }
        }
      }
      __syncthreads();
    }
  }
  for (int i = tid; i < n; i += nt) order[i] = (int64_t)id[i];
}

// Global-memory bitonic stage for key counts that do not fit LDS.
__global__ void argsort_init_kernel(const float* __restrict__ keys, int n, int np2, float* v, int* id) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= np2) return;
  v[i] = (i < n) ? keys[i] : __int_as_float(0x7fc00000);
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
// identity.  Lanes run along i, so reads are coalesced whenever rows are not permuted.
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

template <typename T>
__global__ void copy2d_kernel(const T* __restrict__ in, int64_t ldi, T* __restrict__ out, int64_t ldo, int rows,
                              int cols) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows) return;
  for (int j = blockIdx.y; j < cols; j += gridDim.y) out[i + (int64_t)j * ldo] = in[i + (int64_t)j * ldi];
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
