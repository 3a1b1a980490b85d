// Blocked Householder tridiagonalisation of a dense symmetric matrix (LAPACK sytrd/latrd scheme,
// lower storage), the first stage of the eigensolver that replaces ELPA's one-stage solver
// (src/soap_tp/csrc/elpa_bindings.cpp:149,165).
//
// Per column j of a panel the work falls into four steps, separated by matrix-wide reductions:
//   A  bring column j up to date with the panel's pending rank-2 updates (after finishing the
//      previous w: w += alpha2 v), partial sums of the sub-column norm
//   B  reflector scalars, v, and partial products W^T v, V^T v
//   C  y = A_trailing v : the bandwidth-bound step.  Only the lower triangle is read: a workgroup
//      owns one 128 x 128 tile on or below the diagonal and produces both the tile's product with
//      v (for its rows) and the transposed tile's product (for its columns, a wavefront butterfly
//      per 32 columns); lanes run along rows so every load instruction reads 512 contiguous bytes
//   D  w = tau (y - V (W^T v) - W (V^T v)) and partial sums of w^T v
// Two launches per column: C (trd_symv_kernel, the whole chip) and one fused kernel that runs
// D(j), A(j+1), B(j+1) with a thread per row that keeps its rows of V and W in registers across the
// three steps.  The two reductions inside the fused kernel (w^T v, the norm) travel between its
// workgroups (at most 128, one per 256 rows) as sequence-tagged 64-bit words in device memory,
// like the partial sums of the QR panel kernel; the other reductions cross a launch boundary as
// "write per-workgroup partials, every consumer re-sums them in the same order".  No atomics on
// data, reproducible results.
// The rank-2k update of the trailing matrix runs on the MFMA product over the tiles on or below
// the diagonal only, as one product with K = 64: A -= [V | W] [W | V]^T.
#pragma once
#include "common.hpp"
#include "gemm.hpp"
#include "qr.hpp"

namespace soapmi {

constexpr int kTrdNb = 32;        // panel width
constexpr int kTrdTile = 128;     // tile edge of the matrix-vector product
constexpr int kTrdMaxWg = 128;    // workgroups of the fused column kernel (256 rows each)
constexpr double kTrdReverseAboveBytes = 320.0 * 1024 * 1024;  // see trd_symv_kernel's `reverse`
constexpr int kTrdWideBelow = 256;  // tiles up to which the matrix-vector kernel runs 512 threads per tile (one tile per compute unit)

template <typename T>
struct TrdWorkspace {
  T* vc;        // n x NB   clean reflector block of the current panel (rows are global indices)
  T* w;         // n x NB   directly behind vc: [vc | w] is one n x 2NB operand
  T* vc2;       // n x NB   copy of vc directly behind w: [w | vc2] is the other operand
  T* y_part;    // ceil(n / kTrdTile) x n   one slot per tile that touches an index
  T* dot_part;  // nwg
  T* t_part;    // nwg x 2*NB   partial (W^T v | V^T v)
  unsigned long long* mail;  // 2 reductions x (kTrdMaxWg + 1) values x 2 words
  int* error;   // raised by a workgroup that gave up waiting for a message
};

template <typename T, class WS>
static inline void trd_workspace_layout(WS& ws, int64_t n, TrdWorkspace<T>* out) {
  const int64_t nwg = ceil_div64(n, 256);
  // one allocation, so that the three blocks are adjacent whatever the allocator's alignment is
  T* vc = ws.template take<T>((size_t)3 * n * kTrdNb);
  T* w = vc + (size_t)n * kTrdNb;
  T* vc2 = w + (size_t)n * kTrdNb;
  T* y_part = ws.template take<T>((size_t)n * ceil_div64(n, kTrdTile));
  T* dot_part = ws.template take<T>((size_t)nwg);
  T* t_part = ws.template take<T>((size_t)nwg * 2 * kTrdNb);
  unsigned long long* mail = ws.template take<unsigned long long>(2 * (kTrdMaxWg + 1) * 2 + 2);
  int* error = reinterpret_cast<int*>(mail + 2 * (kTrdMaxWg + 1) * 2);
  if (out) *out = TrdWorkspace<T>{vc, w, vc2, y_part, dot_part, t_part, mail, error};
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

// Sum over the wavefront, in every lane: four steps inside the 16-lane rows on data-parallel-primitive
// moves (partners lane ^ 1, ^ 2, ^ 7, ^ 15), then the rows 16 and 32 lanes apart on the lane-swap
// instructions.  (Six xor-shuffles take six trips through the LDS crossbar, two each for a double.)
template <typename T>
__device__ __forceinline__ T wave_sum_all(T v) {
  v += dpp_partner<kDppQuadXor1>(v);
  v += dpp_partner<kDppQuadXor2>(v);
  v += dpp_partner<kDppRowHalfMirror>(v);
  v += dpp_partner<kDppRowMirror>(v);
  v = swap_add<false>(v, v);
  v = swap_add<true>(v, v);
  return v;
}

// Sum over the 256 threads of a workgroup: each wavefront's sum, then the four wavefront sums in a
// fixed order.  `s_w` is 4 values of shared memory; two barriers.
template <typename T>
__device__ __forceinline__ T block_sum_shuffle(T v, T* s_w) {
  v = wave_sum_all(v);
  __syncthreads();  // earlier readers of s_w are done
  if ((threadIdx.x & 63) == 0) s_w[threadIdx.x >> 6] = v;
  __syncthreads();
  return (s_w[0] + s_w[1]) + (s_w[2] + s_w[3]);
}

// ---- messages between the workgroups of the fused kernel -------------------------------------
// A value travels as one (float) or two (double) 64-bit words {32 payload bits, sequence number},
// each written and read with one single-copy-atomic access: a reader that finds the expected
// sequence number in a word has that word's payload.
__device__ __forceinline__ void mail_post(unsigned long long* slot, float value, unsigned seq) {
  __hip_atomic_store(slot, mailbox_pack(value, seq), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ void mail_post(unsigned long long* slot, double value, unsigned seq) {
  const unsigned lo = (unsigned)__double2loint(value), hi = (unsigned)__double2hiint(value);
  __hip_atomic_store(slot, ((unsigned long long)seq << 32) | lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(slot + 1, ((unsigned long long)seq << 32) | hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Polls until the slot carries `seq`; false after `spin_limit` polls or once `error` is up.
template <typename T>
__device__ __forceinline__ bool mail_fetch(const unsigned long long* slot, unsigned seq, const int* error,
                                           unsigned spin_limit, T* value) {
  constexpr bool WIDE = sizeof(T) == 8;
  unsigned spins = 0;
  for (;;) {
    const unsigned long long w0 = __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned long long w1 =
        WIDE ? __hip_atomic_load(slot + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : w0;
    if ((unsigned)(w0 >> 32) == seq && (unsigned)(w1 >> 32) == seq) {
      if constexpr (WIDE) *value = __hiloint2double((int)(unsigned)w1, (int)(unsigned)w0);
      else *value = __uint_as_float((unsigned)w0);
      return true;
    }
    ++spins;
    if (spins > spin_limit) return false;
    if ((spins & 63u) == 0 && __hip_atomic_load(error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) return false;
    __builtin_amdgcn_s_sleep(1);
  }
}

// Sum of the values posted by `nwg` workgroups (thread t fetches workgroup t's) plus one extra
// value (slot kTrdMaxWg, fetched by thread 255) that comes back in *extra.  All 256 threads call.
// Returns false if a message did not arrive; `s_fail` and `s_x` are shared scratch.
template <typename T>
__device__ __forceinline__ bool mail_gather(const unsigned long long* mail, int nwg, unsigned seq, int* error,
                                            unsigned spin_limit, T* s_w, T* s_x, int* s_fail, T* sum, T* extra) {
  const int tid = threadIdx.x;
  T v = T(0);
  bool ok = true;
  if (tid < nwg) ok = mail_fetch<T>(mail + 2 * tid, seq, error, spin_limit, &v);
  if (tid == 255) {
    T x = T(0);
    ok = mail_fetch<T>(mail + 2 * kTrdMaxWg, seq, error, spin_limit, &x);
    *s_x = x;
  }
  if (!ok) {
    __hip_atomic_store(error, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *s_fail = 1;
  }
  *sum = block_sum_shuffle(v, s_w);  // its barriers also publish s_x and s_fail
  *extra = *s_x;
  return *s_fail == 0;
}

// W[r, col] += alpha2 * Vc[r, col] for rows r >= row0: the last w of a panel, which no later
// column step finishes, before the rank-2k update reads it.
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

// Steps D(j), A(jn), B(jn) with jn = j + 1, one thread per row r = jn + 256 * workgroup + thread.
//   do_d    : step D runs (j is a column of this panel whose v and y exist); otherwise the launch
//             opens a panel at column jn = p and only A and B run
//   do_next : steps A and B run (jn is still inside the panel); otherwise the launch ends after D
//             and leaves the unfinished w and the partial sums of w^T v for trd_finish_w_kernel
// i = j - p is the index of reflector j in the panel; columns k < i of Vc and W are final in memory,
// column i of W is produced here.  `n_t_part` is the grid size of the launch that ran B(j).
// `seq` (unique per launch, never 0) tags this launch's messages.
template <typename T>
__global__ __launch_bounds__(256) void trd_column_kernel(T* __restrict__ A, int64_t lda, int n, int p, int j,
                                                         int do_d, int do_next, T* __restrict__ Vc,
                                                         T* __restrict__ Vc2, T* __restrict__ W, int64_t ldw,
                                                         const T* __restrict__ y_part, int n_slots,
                                                         T* __restrict__ t_part, int n_t_part,
                                                         T* __restrict__ dot_part, T* __restrict__ tau,
                                                         T* __restrict__ d, T* __restrict__ e,
                                                         unsigned long long* mail, unsigned seq, int* error,
                                                         unsigned spin_limit) {
  constexpr int NB = kTrdNb;
  __shared__ T s_t[2 * NB];
  __shared__ T s_t4[4][2 * NB];
  __shared__ T s_wj[NB], s_vj[NB];
  __shared__ T s_red[4][2 * NB];
  __shared__ T s_row[2 * NB];  // row jn + 1 of [W | Vc] (columns up to i), written by its owner in workgroup 0
  __shared__ T s_w4[4];
  __shared__ T s_x;
  __shared__ int s_fail;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int nwg = gridDim.x, wg = blockIdx.x;
  const int jn = j + 1;
  const int i = j - p;  // valid when do_d
  const int r = jn + wg * 256 + tid;
  const bool live = r < n;
  unsigned long long* mail_dot = mail;
  unsigned long long* mail_norm = mail + 2 * (kTrdMaxWg + 1);
  if (tid == 0) s_fail = 0;

  T vr[NB], wr[NB];  // this row of Vc and W, columns k < i
#pragma unroll
  for (int k = 0; k < NB; ++k) vr[k] = wr[k] = T(0);
  T vi = T(0), wv = T(0);  // this row of column i: v_j and the unfinished w_j
  T alpha2 = T(0), w_jn_i = T(0);
  T acc_old = T(0), a_loaded = T(0);

  if (do_d) {
    // ---- D(j): w = tau (y - V (W^T v) - W (V^T v)) ----
    // This row of the panel's finished columns and of y first: the loads are on their way while the
    // partial products of the launch before are summed.
    T y = T(0);
    if (live) {
#pragma unroll
      for (int k = 0; k < NB; ++k) {
        vr[k] = (k < i) ? Vc[r + (int64_t)k * ldw] : T(0);
        wr[k] = (k < i) ? W[r + (int64_t)k * ldw] : T(0);
      }
      vi = Vc[r + (int64_t)i * ldw];
      for (int c0 = 0; c0 < n_slots; c0 += 32) {  // 32 slot loads in flight, summed in slot order
        T yp[32];
#pragma unroll
        for (int c = 0; c < 32; ++c) yp[c] = (c0 + c < n_slots) ? y_part[(int64_t)(c0 + c) * n + r] : T(0);
#pragma unroll
        for (int c = 0; c < 32; ++c) y += yp[c];
      }
    }
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
    if (live) {
      T corr = T(0);
#pragma unroll
      for (int k = 0; k < NB; ++k) corr += vr[k] * s_t[k] + wr[k] * s_t[NB + k];
      wv = tau[j] * (y - corr);
      prod = wv * vi;
    }
    const T dot = block_sum_shuffle(prod, s_w4);
    if (!do_next) {
      if (live) W[r + (int64_t)i * ldw] = wv;
      if (tid == 0) dot_part[wg] = dot;
      return;
    }
    if (tid == 0) mail_post(mail_dot + 2 * wg, dot, seq);
    if (r == jn) mail_post(mail_dot + 2 * kTrdMaxWg, wv, seq);  // the unfinished W[jn, i]
    // While the messages travel: what the finished columns k < i contribute to the update of column
    // jn (row jn of those columns is final in memory), and column jn itself.
    if (tid < i) {
      s_wj[tid] = W[jn + (int64_t)tid * ldw];
      s_vj[tid] = Vc[jn + (int64_t)tid * ldw];
    }
    if (live) a_loaded = A[r + (int64_t)jn * lda];
    __syncthreads();
#pragma unroll
    for (int k = 0; k < NB; ++k)
      if (k < i) acc_old += vr[k] * s_wj[k] + wr[k] * s_vj[k];
    T total, w_jn_raw;
    if (!mail_gather<T>(mail_dot, nwg, seq, error, spin_limit, s_w4, &s_x, &s_fail, &total, &w_jn_raw)) return;
    alpha2 = T(-0.5) * tau[j] * total;
    w_jn_i = w_jn_raw + alpha2;  // v_j has its unit entry in row jn
  } else if (live) {
    a_loaded = A[r + (int64_t)jn * lda];
  }

  // ---- A(jn): finish w_j, bring column jn up to date, norm of its sub-column ----
  const int in = jn - p;  // reflectors in the panel before column jn
  T wf = T(0);
  if (do_d) {
    wf = wv + alpha2 * vi;
    if (live) W[r + (int64_t)i * ldw] = wf;
  }
  T a = T(0), x2 = T(0);
  if (live) {
    a = a_loaded;
    if (do_d) {
      // column i: Vc[r,i] W[jn,i] + W[r,i] Vc[jn,i], Vc[jn,i] = 1
      a -= (vi * w_jn_i + wf) + acc_old;
      A[r + (int64_t)jn * lda] = a;
    }
    if (r == jn) d[jn] = a;
    if (r > jn + 1) x2 = a * a;
  }
  if (jn >= n - 1) return;  // the last column has no reflector
  const T norm_part = block_sum_shuffle(x2, s_w4);
  if (tid == 0) mail_post(mail_norm + 2 * wg, norm_part, seq);
  if (r == jn + 1) mail_post(mail_norm + 2 * kTrdMaxWg, a, seq);  // alpha
  // While the messages travel: v = scale * a below row jn + 1, so this workgroup's part of W^T v
  // and V^T v is scale times its part of W^T a and V^T a over those rows, plus row jn + 1 itself
  // (where v = 1); the sums over the rows are formed now and scaled once `scale` is known.
  {
    const T u = (live && r > jn + 1) ? a : T(0);
    T pw[NB], pv[NB];
#pragma unroll
    for (int k = 0; k < NB; ++k) {
      const T wk = (do_d && k == i) ? wf : wr[k];  // wr, vr are zero beyond column i
      const T vk = (do_d && k == i) ? vi : vr[k];
      pw[k] = wk * u;
      pv[k] = vk * u;
      if (r == jn + 1) {  // (one thread of workgroup 0)
        s_row[k] = wk;
        s_row[NB + k] = vk;
      }
    }
    const T tw = wave_reduce_32<T>(pw, lane);
    const T tv = wave_reduce_32<T>(pv, lane);
    if ((lane & 1) == 0) {
      s_red[wave][(lane >> 1) & 31] = tw;
      s_red[wave][NB + ((lane >> 1) & 31)] = tv;
    }
  }
  T x2_total, alpha;
  if (!mail_gather<T>(mail_norm, nwg, seq, error, spin_limit, s_w4, &s_x, &s_fail, &x2_total, &alpha)) return;

  // ---- B(jn): reflector, v, partial W^T v and V^T v ----
  T beta = alpha, tauv = T(0), scale = T(0);
  if (x2_total > T(0)) {
    const T nrm = sqrt(alpha * alpha + x2_total);
    beta = (alpha >= T(0)) ? -nrm : nrm;
    tauv = (beta - alpha) / beta;
    scale = T(1) / (alpha - beta);
  }
  T v = T(0);
  if (live && r > jn) {
    if (r == jn + 1) {
      v = T(1);
      tau[jn] = tauv;
      e[jn] = beta;
    } else {
      v = a * scale;
      A[r + (int64_t)jn * lda] = v;  // reflector kept for the back-transformation
    }
  }
  if (live) {  // row jn reads as zero, like the rows above it
    Vc[r + (int64_t)in * ldw] = v;
    Vc2[r + (int64_t)in * ldw] = v;
  }
  if (wg == 0) {
    for (int rr = p + tid; rr < jn; rr += 256) {
      Vc[rr + (int64_t)in * ldw] = T(0);
      Vc2[rr + (int64_t)in * ldw] = T(0);
    }
  }
  // (s_red and s_row were written before the wait; the barriers of mail_gather lie in between)
  if (tid < 2 * NB) {
    const T below = (s_red[0][tid] + s_red[1][tid]) + (s_red[2][tid] + s_red[3][tid]);
    const bool has_row = wg == 0 && jn + 1 < n;  // row jn + 1 is row 1 of workgroup 0
    t_part[(int64_t)wg * 2 * NB + tid] = scale * below + (has_row ? s_row[tid] : T(0));
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
// QS = 1: 256 threads, a thread takes its row's 64 entries in two groups of 32 columns, one after
// the other.  QS = 2: 512 threads, the two groups go to two sets of four wavefronts, so that a tile
// is one trip to memory and one round of arithmetic instead of two each; the host picks it while
// there are no more tiles than compute units (there the chain of one tile is the time of the launch;
// a compute unit holds one such workgroup), and QS = 1, three tiles per compute unit, above.
template <typename T, int QS>
__global__ __launch_bounds__(256 * QS) void trd_symv_kernel(const T* __restrict__ A, int64_t lda, int n, int j,
                                                            const T* __restrict__ v, T* __restrict__ y_part,
                                                            int reverse) {
  constexpr int TS = kTrdTile;
  __shared__ T s_v[TS];
  __shared__ T s_direct[2 * QS][TS];
  __shared__ T s_col[4][64];
  const int tid = threadIdx.x & 255, lane = tid & 63, wave = tid >> 6;
  const int q_first = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 8);  // 0 unless QS = 2
  // `half` is the same for all lanes of a wavefront: telling the compiler so moves the column
  // address arithmetic to the scalar unit
  const int row = tid & (TS - 1), half = __builtin_amdgcn_readfirstlane(tid >> 7);
  const int o = j + 1;
  // Workgroups start in the order of their ids.  Every other column walks the tiles backwards: the
  // tiles a launch touches last are the ones most likely still held by the 256 MB memory-side cache
  // when the next column's launch, whose tiles are the same memory shifted by one row and column,
  // begins with them.  (Walking forwards every time, a matrix larger than that cache evicts the
  // head of the walk before the next launch comes back to it.)
  const int t = reverse ? (int)gridDim.x - 1 - (int)blockIdx.x : (int)blockIdx.x;
  int rb = (int)((sqrtf(8.0f * (float)t + 1.0f) - 1.0f) * 0.5f);
  while (rb * (rb + 1) / 2 > t) --rb;
  while ((rb + 1) * (rb + 2) / 2 <= t) ++rb;
  const int cb = t - rb * (rb + 1) / 2;
  const int r = o + rb * TS + row;        // global row of this thread
  const int c0 = o + cb * TS;             // first global column of the tile
  const bool live = r < n;
  const bool diagonal = rb == cb;
  T vr = T(0);
  T acc0 = T(0), acc1 = T(0);
  // Loads are unconditional on clamped addresses (always inside the matrix); what must not count
  // - rows past the end, the upper triangle inside a diagonal tile - is zeroed after the load.
  const int rr = min(r, n - 1);
  const int limit = diagonal ? r : n - 1;  // last column that counts for this row
#pragma unroll 1
  for (int q = q_first; q < 2; q += QS) {  // 32 columns at a time
    const int cq = c0 + 64 * half + 32 * q;
    T a[32];
#pragma unroll
    for (int k = 0; k < 32; ++k) a[k] = A[rr + (int64_t)min(cq + k, n - 1) * lda];
    if (q == q_first) {
      // The tile's piece of v is requested behind the first 32 columns and published by a barrier
      // that waits for both: one trip to memory instead of two (from about 4 000 rows down a
      // compute unit has one tile or none, and the trips are the time).
      if (threadIdx.x < TS) s_v[threadIdx.x] = (c0 + (int)threadIdx.x < n) ? v[c0 + threadIdx.x] : T(0);
      vr = live ? v[r] : T(0);
      __syncthreads();
    }
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
  s_direct[2 * q_first + half][row] = acc0 + acc1;
  __syncthreads();
  if (threadIdx.x < TS) {
    // wavefronts 2*half and 2*half+1 (of either set) hold the two row halves of column half `half`
    const int h = tid >> 6, k = tid & 63;
    const T column_sum = s_col[2 * h][k] + s_col[2 * h + 1][k];
    T row_sum = s_direct[0][tid] + s_direct[1][tid];
    if constexpr (QS == 2) row_sum += s_direct[2][tid] + s_direct[3][tid];
    const int gr = o + rb * TS + tid, gc = c0 + tid;
    if (diagonal) {
      if (gr < n) y_part[(int64_t)rb * n + gr] = row_sum + column_sum;
    } else {
      if (gr < n) y_part[(int64_t)cb * n + gr] = row_sum;
      if (gc < n) y_part[(int64_t)rb * n + gc] = column_sum;
    }
  }
}

// Tridiagonalise A (n x n, lower triangle referenced; destroyed).  On exit d[0..n), e[0..n-1),
// tau[0..n-1) and, below the first subdiagonal of A, the reflector vectors (implicit unit at
// row j+1 of column j), as LAPACK sytrd('L') leaves them.  *ws.error is nonzero afterwards if a
// workgroup of the column kernel gave up waiting for a message; the results are then unusable and
// the caller has to make that visible.
template <typename T>
static inline int sytrd_lower(hipStream_t s, T* A, int64_t lda, int n, T* d, T* e, T* tau, const TrdWorkspace<T>& ws,
                              unsigned spin_limit = kQrSpinLimit) {
  constexpr int NB = kTrdNb;
  const int64_t ldw = n;
  if (n == 1) {
    SOAPMI_HIP(hipMemcpyAsync(d, A, sizeof(T), hipMemcpyDeviceToDevice, s));
    return kOk;
  }
  SOAPMI_REQUIRE(ceil_div64(n, 256) <= kTrdMaxWg, "matrix size %d exceeds what the column kernel supports", n);
  {
    // messages of an earlier factorisation in the same workspace must not be mistaken for new ones
    const int words = 2 * (2 * (kTrdMaxWg + 1) * 2 + 2);
    hipLaunchKernelGGL((fill_zero_kernel<unsigned>), dim3((words + 255) / 256), dim3(256), 0, s,
                       reinterpret_cast<unsigned*>(ws.mail), words);
  }
  unsigned seq = 0;
  for (int p = 0; p < n; p += NB) {
    const int pe = std::min(n, p + NB);
    // open the panel: A(p), B(p)
    int grid = (int)ceil_div64(n - p, 256);
    hipLaunchKernelGGL((trd_column_kernel<T>), dim3(grid), dim3(256), 0, s, A, lda, n, p, p - 1, 0, 1, ws.vc, ws.vc2,
                       ws.w, ldw, ws.y_part, 0, ws.t_part, 0, ws.dot_part, tau, d, e, ws.mail, ++seq, ws.error,
                       spin_limit);
    int t_parts = grid;  // grid of the launch that ran B for the current column
    int cols_done = 0, last_dot_parts = 0;
    for (int j = p; j < pe; ++j) {
      if (j == n - 1) break;  // only the diagonal entry remained, and A(n-1) has stored it
      const int i = j - p;
      const int nt = n - j - 1;
      const int nb = (int)ceil_div64(nt, kTrdTile);
      // (backwards on every other column while the triangle that is read is larger than the memory-side
      // cache: measured 662 -> 646 ms at n = 11008 and 1297 -> 1263 ms at 14336 in fp64; below that size
      // it costs 1 to 2 %)
      const int reverse = ((j & 1) != 0 && (double)nt * (double)nt * 0.5 * sizeof(T) > kTrdReverseAboveBytes) ? 1 : 0;
      if (nb * (nb + 1) / 2 <= kTrdWideBelow)
        hipLaunchKernelGGL((trd_symv_kernel<T, 2>), dim3(nb * (nb + 1) / 2), dim3(512), 0, s, A, lda, n, j,
                           ws.vc + (int64_t)i * ldw, ws.y_part, reverse);
      else
        hipLaunchKernelGGL((trd_symv_kernel<T, 1>), dim3(nb * (nb + 1) / 2), dim3(256), 0, s, A, lda, n, j,
                           ws.vc + (int64_t)i * ldw, ws.y_part, reverse);
      grid = (int)ceil_div64(nt, 256);
      const int do_next = (j + 1 < pe) ? 1 : 0;
      hipLaunchKernelGGL((trd_column_kernel<T>), dim3(grid), dim3(256), 0, s, A, lda, n, p, j, 1, do_next, ws.vc, ws.vc2,
                         ws.w, ldw, ws.y_part, nb, ws.t_part, t_parts, ws.dot_part, tau, d, e, ws.mail, ++seq,
                         ws.error, spin_limit);
      t_parts = grid;
      last_dot_parts = grid;
      cols_done = i + 1;
    }
    SOAPMI_LAUNCH_CHECK();
    if (pe >= n) break;
    // finish the last w of the panel, then A[pe:, pe:] -= [V | W] [W | V]^T on the lower tiles
    const int jl = pe - 1;
    hipLaunchKernelGGL((trd_finish_w_kernel<T>), dim3((unsigned)ceil_div64(n - pe, 256)), dim3(256), 0, s, ws.w, ws.vc,
                       ldw, n, pe, cols_done - 1, ws.dot_part, last_dot_parts, tau + jl);
    const int nt = n - pe;
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
