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
// that both the reads and the writes are coalesced.
template <typename T>
__global__ void transpose_kernel(const T* __restrict__ in, int64_t ldi, T* __restrict__ out, int64_t ldo, int R,
                                 int C) {
  __shared__ T tile[64][65];
  const int r0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
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
