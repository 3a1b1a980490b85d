// Bandwidth-bound helper kernels: Adam, layout transposes, symmetrisation, gathers, column dots.
#pragma once
#include "common.hpp"
#include "gemm.hpp"

namespace soapmi {

// One thread per element, lanes along the contiguous (row) index of the column-major buffers.
__global__ void adam_kernel(const float* __restrict__ g, int64_t ldg, float* mom, int64_t ldm, float* var,
                            int64_t ldv, float* upd, int64_t ldu, int rows, int cols, AdamScalars s) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows) return;
  for (int j = blockIdx.y; j < cols; j += gridDim.y) {
    float gv = g[i + (int64_t)j * ldg];
    upd[i + (int64_t)j * ldu] = adam_element(gv, mom + i + (int64_t)j * ldm, var + i + (int64_t)j * ldv, s);
  }
}

// out[c + r*ldo] = in[r + c*ldi] for an R x C column-major `in`: a 64x64 tile goes through LDS so
// that both the reads and the writes are coalesced.  With `vec` (both buffers 16-byte aligned with
// leading dimensions and extents that are multiples of the vector width) every global access moves
// 16 bytes.
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(const T* __restrict__ in, int64_t ldi, T* __restrict__ out,
                                                        int64_t ldo, int R, int C, int vec = 0) {
  constexpr int VW = Vec16<T>::W;
  using V = typename Vec16<T>::type;
  __shared__ T tile[64][65];
  const int r0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
  if (vec) {
    constexpr int PER = 64 / VW;  // vectors along a tile edge
    for (int e = threadIdx.x; e < 64 * PER; e += 256) {
      const int c = e / PER, rv = (e % PER) * VW;
      const int gr = r0 + rv, gc = c0 + c;
      if (gr < R && gc < C) {
        const V t = *reinterpret_cast<const V*>(in + gr + (int64_t)gc * ldi);
        const T* tp = reinterpret_cast<const T*>(&t);
#pragma unroll
        for (int q = 0; q < VW; ++q) tile[c][rv + q] = tp[q];
      }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < 64 * PER; e += 256) {
      const int r = e / PER, cv = (e % PER) * VW;
      const int gr = r0 + r, gc = c0 + cv;
      if (gr < R && gc < C) {
        V t;
        T* tp = reinterpret_cast<T*>(&t);
#pragma unroll
        for (int q = 0; q < VW; ++q) tp[q] = tile[cv + q][r];
        *reinterpret_cast<V*>(out + gc + (int64_t)gr * ldo) = t;
      }
    }
    return;
  }
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 256 threads: 64 x 4
  for (int c = ty; c < 64; c += 4) {
    int gr = r0 + tx, gc = c0 + c;
    if (gr < R && gc < C) tile[c][tx] = in[gr + (int64_t)gc * ldi];
  }
  __syncthreads();
  for (int r = ty; r < 64; r += 4) {
    int gc = c0 + tx, gr = r0 + r;
    if (gr < R && gc < C) out[gc + (int64_t)gr * ldo] = tile[tx][r];
  }
}

// Whether transpose_kernel may use 16-byte accesses for this pair of buffers.
template <typename T>
static inline int transpose_vec_ok(const T* in, int64_t ldi, const T* out, int64_t ldo, int64_t R, int64_t C) {
  constexpr int VW = Vec16<T>::W;
  return reinterpret_cast<uintptr_t>(in) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 && ldi % VW == 0 &&
         ldo % VW == 0 && R % VW == 0 && C % VW == 0;
}

// Upper triangle <- transpose of the strictly lower triangle.  One workgroup per 64x64 tile on or
// below the diagonal (tiles above it return at once).
template <typename T>
__global__ void symmetrize_lower_kernel(T* p, int64_t ld, int n) {
  __shared__ T tile[64][65];
  const int bi = blockIdx.x, bj = blockIdx.y;
  if (bi < bj) return;
  const int r0 = bi * 64, c0 = bj * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int c = ty; c < 64; c += 4) {
    int gr = r0 + tx, gc = c0 + c;
    if (gr < n && gc < n) tile[c][tx] = p[gr + (int64_t)gc * ld];
  }
  __syncthreads();
  for (int r = ty; r < 64; r += 4) {
    // element (row gr = r0 + r, col gc = c0 + tx) of the lower tile goes to (gc, gr)
    int gr = r0 + r, gc = c0 + tx;
    if (gr < n && gc < n && gr > gc) p[gc + (int64_t)gr * ld] = tile[tx][r];
  }
}

}  // namespace soapmi
