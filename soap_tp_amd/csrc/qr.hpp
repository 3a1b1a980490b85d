// Blocked Householder QR (LAPACK geqrf sign convention) and explicit formation of Q, for the
// power-iteration refresh of a SOAP eigenbasis (what the reference obtains from SLATE's
// geqrf + unmqr on the identity: src/soap_tp/csrc/slate_bindings.cpp:176-185).
//
// Panel (NB = 32 columns): a workgroup owns 256 rows, one per thread, and keeps its row of the
// panel in registers.  Normally the whole panel runs in one persistent launch whose workgroups
// exchange partial dot products through device memory, two columns per exchange
// (qr_panel_persistent_kernel); beyond kQrPersistentMaxWg workgroups it runs one launch per column
// (qr_panel_step_kernel: launch j applies reflector j, whose dot products with the remaining
// panel columns were reduced by launch j-1, and in the same pass reduces the dot products reflector
// j+1 needs).  Reductions are a 32-value butterfly over the wavefront, then a fixed-order sum over
// workgroups: no atomics on data, so results do not depend on scheduling.
// Trailing matrix and Q formation: compact-WY block reflectors on the MFMA GEMM.
#pragma once
#include <type_traits>

#include "common.hpp"
#include "gemm.hpp"

namespace soapmi {

constexpr int kQrNb = 32;

// One butterfly stage: lanes whose bit MASK is set keep the upper HALF values, the others the
// lower HALF, and each adds what its partner (lane ^ MASK) holds for the same positions.
template <typename T, int HALF, int MASK>
__device__ __forceinline__ void butterfly_stage(T (&vals)[32], int lane) {
  const bool upper = (lane & MASK) != 0;
#pragma unroll
  for (int c = 0; c < HALF; ++c) {
    const T send = upper ? vals[c] : vals[c + HALF];
    const T keep = upper ? vals[c + HALF] : vals[c];
    vals[c] = keep + __shfl_xor(send, MASK, 64);
  }
}

// The two widest stages (partners 32 and 16 lanes apart) on gfx950's lane-swap instructions:
// v_permlane32_swap exchanges lanes 32..63 of its first operand with lanes 0..31 of its second
// (v_permlane16_swap: the odd 16-lane rows of the first with the even rows of the second), which is
// exactly "send the half I do not keep, receive the half I keep": afterwards the two registers hold
// the two addends in every lane, with no select and no trip through the LDS crossbar.
template <bool WIDE32>
__device__ __forceinline__ void lane_swap(unsigned& a, unsigned& b) {
  if constexpr (WIDE32) {
    const auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
    a = r[0];
    b = r[1];
  } else {
    const auto r = __builtin_amdgcn_permlane16_swap(a, b, false, false);
    a = r[0];
    b = r[1];
  }
}

template <bool WIDE32>
__device__ __forceinline__ float swap_add(float a, float b) {
  unsigned ua = __float_as_uint(a), ub = __float_as_uint(b);
  lane_swap<WIDE32>(ua, ub);
  return __uint_as_float(ua) + __uint_as_float(ub);
}

template <bool WIDE32>
__device__ __forceinline__ double swap_add(double a, double b) {
  unsigned a_lo = (unsigned)__double2loint(a), a_hi = (unsigned)__double2hiint(a);
  unsigned b_lo = (unsigned)__double2loint(b), b_hi = (unsigned)__double2hiint(b);
  lane_swap<WIDE32>(a_lo, b_lo);
  lane_swap<WIDE32>(a_hi, b_hi);
  return __hiloint2double((int)a_hi, (int)a_lo) + __hiloint2double((int)b_hi, (int)b_lo);
}

template <typename T, int HALF, bool WIDE32>
__device__ __forceinline__ void butterfly_stage_swap(T (&vals)[32]) {
#pragma unroll
  for (int c = 0; c < HALF; ++c) vals[c] = swap_add<WIDE32>(vals[c], vals[c + HALF]);
}

// After the call lane l holds, in the return value, the sum over the wavefront of vals[(l>>1)&31].
// Stages are spelled out so that every register index is a compile-time constant.
template <typename T>
__device__ __forceinline__ T wave_reduce_32(T (&vals)[32], int lane) {
  butterfly_stage_swap<T, 16, true>(vals);
  butterfly_stage_swap<T, 8, false>(vals);
  butterfly_stage<T, 4, 8>(vals, lane);
  butterfly_stage<T, 2, 4>(vals, lane);
  butterfly_stage<T, 1, 2>(vals, lane);
  return vals[0] + __shfl_xor(vals[0], 1, 64);
}

template <typename T>
__global__ __launch_bounds__(256) void qr_panel_step_kernel(T* __restrict__ A, int64_t lda, int n, int p, int pe, int j,
                                                            const T* __restrict__ part_in,
                                                            const T* __restrict__ piv_in, T* __restrict__ part_out,
                                                            T* __restrict__ piv_out, T* __restrict__ tau, int nwg) {
  constexpr int NB = kQrNb;
  __shared__ T s_tc[NB];
  __shared__ T s_wave[4][NB];
  __shared__ T s_sum8[8][NB];
  __shared__ T s_piv[NB];
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
    {
      // fixed-order sum of the per-workgroup partials: 8 strided partial sums per column, then 8 adds
      const int c = tid & (NB - 1), g = tid >> 5;
      T s = T(0);
      for (int w0 = g; w0 < nwg; w0 += 64) {
        T v[8];  // eight independent loads in flight, then a fixed-order sum
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = (w0 + 8 * u < nwg) ? part_in[(w0 + 8 * u) * NB + c] : T(0);
#pragma unroll
        for (int u = 0; u < 8; ++u) s += v[u];
      }
      s_sum8[g][c] = s;
      if (tid < NB) s_piv[tid] = (tid < ncol) ? piv_in[tid] : T(0);
    }
    __syncthreads();
    if (tid < NB) {
      // every one of these lanes derives the reflector scalars from the same sums
      T x2 = T(0), dot = T(0);
#pragma unroll
      for (int g = 0; g < 8; ++g) {
        x2 += s_sum8[g][0];
        dot += s_sum8[g][tid];
      }
      const T alpha = s_piv[0];
      T beta = alpha, tauv = T(0), scale = T(0);
      if (x2 > T(0)) {
        const T nrm = sqrt(alpha * alpha + x2);
        beta = (alpha >= T(0)) ? -nrm : nrm;
        tauv = (beta - alpha) / beta;
        scale = T(1) / (alpha - beta);
      }
      s_tc[tid] = (tid >= 1 && tid < ncol) ? tauv * (s_piv[tid] + scale * dot) : T(0);
      if (tid == 0) {
        s_scal[0] = scale; s_scal[1] = beta; s_scal[2] = tauv;
      }
    }
    __syncthreads();
    const T scale = s_scal[0], beta = s_scal[1], tauv = s_scal[2];
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

// ---- whole panel in one launch -----------------------------------------------------------------
// The same column recurrence as qr_panel_step_kernel, but the 32 columns of a panel run inside
// one launch: every thread keeps its row of the panel in registers from the first column to the
// last (loaded once, each finished column stored once).  Between columns the workgroups exchange
// their partial dot products (and the pivot row) through "mailbox" words in device memory: every
// value travels as one 64-bit word {float bits, sequence number} written and read with single-copy
// atomic accesses, so a reader that sees the expected sequence number has the value with it.  No
// separate flag, counter or fence is needed, and a column costs one trip through memory.
// Sequence numbers grow by one per message round over the whole factorisation (the host passes
// the launch's starting value and clears the mailboxes before the first panel), mailboxes
// alternate between two sets by round parity: a workgroup writes round t+2 only after it has read
// every workgroup's round t+1, which those wrote after they had read round t.
// Besides A the kernel writes the panel's reflectors in clean form (unit diagonal, zeros above) to
// vout, the operand of the block-reflector products.
// Requirements: all workgroups of the launch are resident at the same time (the host launches at
// most kQrPersistentMaxWg of them, one per CU).  Waiting is bounded: a thread that does not see a
// word arrive within `spin_limit` polls (kQrSpinLimit unless the caller lowers it) raises `error`, and every workgroup that sees the flag or
// runs out of patience itself leaves the kernel.
constexpr int kQrPersistentMaxWg = 128;
constexpr unsigned kQrSpinLimit = 1u << 22;

__device__ __forceinline__ unsigned long long mailbox_pack(float value, unsigned seq) {
  return ((unsigned long long)seq << 32) | (unsigned long long)__float_as_uint(value);
}

// Reads COUNT mailbox words until all carry `seq`; false after too many polls or once the error
// flag is up.
template <int COUNT>
__device__ __forceinline__ bool mailbox_wait(const unsigned long long* const (&slot)[COUNT], const bool (&used)[COUNT],
                                             unsigned seq, const int* error, unsigned spin_limit,
                                             float (&value)[COUNT]) {
  unsigned spins = 0;
  for (;;) {
    unsigned long long word[COUNT];
#pragma unroll
    for (int u = 0; u < COUNT; ++u)
      word[u] = used[u] ? __hip_atomic_load(slot[u], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                        : mailbox_pack(0.0f, seq);
    bool ready = true;
#pragma unroll
    for (int u = 0; u < COUNT; ++u) ready = ready && (unsigned)(word[u] >> 32) == seq;
    if (ready) {
#pragma unroll
      for (int u = 0; u < COUNT; ++u) value[u] = __uint_as_float((unsigned)word[u]);
      return true;
    }
    ++spins;
    if (spins > spin_limit) return false;
    if ((spins & 63u) == 0 && __hip_atomic_load(error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) return false;
    __builtin_amdgcn_s_sleep(1);
  }
}

// Householder scalars of a column with leading entry alpha and squared norm x2 of the rest.
// A column whose squared norm is at most `floor2` is left alone (tau = 0): see kQrNegligible.
struct Reflector {
  float beta, tau, scale;
};
__device__ __forceinline__ Reflector make_reflector(float alpha, float x2, float floor2) {
  Reflector h{alpha, 0.0f, 0.0f};
  if (x2 > 0.0f && alpha * alpha + x2 > floor2) {
    const float nrm = sqrtf(alpha * alpha + x2);
    h.beta = (alpha >= 0.0f) ? -nrm : nrm;
    h.tau = (h.beta - alpha) / h.beta;
    h.scale = 1.0f / (alpha - h.beta);
  }
  return h;
}

// A column whose squared norm has fallen below kQrNegligible times the largest one met so far in
// its panel (a norm ratio of 1e-12) gets no reflector.  Such columns are rounding residue of
// exactly dependent columns; left to themselves they shrink by 1e-7 per column until their
// squares underflow, and a reflector built from underflowed sums is not orthogonal (LAPACK's
// slarfg rescales instead, which a norm that comes out of a reduction cannot do in place).
// What stays below the diagonal of R is below 1e-12 of the panel's scale; Q stays orthogonal.
constexpr float kQrNegligible = 1e-24f;

// Two columns per message round.  Besides the dot products of column j with the remaining columns
// (over the rows below the pivot) a round also reduces those of column j+1 as it stands (over the
// rows below ITS pivot) and broadcasts both pivot rows.  Once reflector j is known, what column
// j+1 and its dot products become after applying it follows by a rank-one correction,
//   a'_k = a_k - tc_k v,  <a'_1, a'_k> = <a_1, a_k> - tc_k s <a_0, a_1> - tc_1 s <a_0, a_k> + tc_1 tc_k s^2 <a_0, a_0>
// (s = reflector j's scale, sums over the rows below pivot j+1), so reflector j+1 needs no second
// round.  The corrected squared norm of column j+1 is a difference: when it comes out below
// kQrPairGuard times the size of the terms it is formed from (column j+1 nearly parallel to
// column j, cancellation), the pair is abandoned, only reflector j is applied, and column j+1 gets a round of its own with
// directly computed sums.  Every workgroup takes that decision from the same numbers.
constexpr float kQrPairGuard = 0.25f;

__global__ __launch_bounds__(256) void qr_panel_persistent_kernel(float* __restrict__ A, int64_t lda, int n, int p,
                                                                  int pe, unsigned long long* part,
                                                                  unsigned long long* piv, float* __restrict__ tau,
                                                                  unsigned seq_base, int* error, int nwg,
                                                                  unsigned spin_limit, float* __restrict__ vout,
                                                                  int64_t ldv, int vrow0, int pairs) {
  using T = float;
  constexpr int NB = kQrNb;
  __shared__ T s_wave[4][2 * NB];
  __shared__ T s_sum4[4][2 * NB];
  __shared__ T s_piv_out[2 * NB];
  __shared__ T s_tot[2 * NB];   // [0, NB): column j's sums, [NB, 2 NB): column j+1's
  __shared__ T s_piv[2 * NB];   // pivot rows j and j+1
  __shared__ T s_tc[2][NB];
  __shared__ T s_scal[8];
  __shared__ int s_pair_ok;
  __shared__ int s_fail;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wg = blockIdx.x;
  const int r = p + wg * 256 + tid;
  const int nbw = pe - p;
  const bool live = r < n;
  if (tid == 0) {
    s_fail = 0;
    s_scal[6] = T(0);
  }
  // vout (rows vrow0.., one column per panel column) receives the reflectors in clean form: zeros
  // above the unit diagonal, including the vrow0 - p ... rows above the panel that no thread owns
  if (wg == 0) {
    for (int t = tid; t < (p - vrow0) * nbw; t += 256) vout[t % (p - vrow0) + (int64_t)(t / (p - vrow0)) * ldv] = T(0);
  }

  T a[NB];  // a[k] = A[r, j + k] for the current column j: the row is shifted left after each column
#pragma unroll
  for (int c = 0; c < NB; ++c) a[c] = (live && c < nbw) ? A[r + (int64_t)(p + c) * lda] : T(0);

  int c = 0;
  for (unsigned round = 0; c < nbw; ++round) {
    const int j = p + c;
    const bool pair = pairs != 0 && c + 1 < nbw;
    const int width = pair ? 2 * NB : NB;  // values per workgroup in this round
    const unsigned seq = seq_base + round + 1u;
    unsigned long long* part_c = part + (size_t)(round & 1) * kQrPersistentMaxWg * 2 * NB;
    unsigned long long* piv_c = piv + (round & 1) * 2 * NB;
    // dot products over the rows below the pivot(s)
    {
      const bool below = live && r > j;
      T vals[NB];
#pragma unroll
      for (int k = 0; k < NB; ++k) vals[k] = below ? a[0] * a[k] : T(0);
      const T total = wave_reduce_32<T>(vals, lane);
      if ((lane & 1) == 0) s_wave[wave][(lane >> 1) & 31] = total;
      if (live && r == j) {
#pragma unroll
        for (int k = 0; k < NB; ++k) s_piv_out[k] = a[k];
      }
    }
    if (pair) {
      const bool below = live && r > j + 1;
      T vals[NB];
#pragma unroll
      for (int k = 0; k < NB; ++k) vals[k] = below ? a[1] * a[k] : T(0);
      const T total = wave_reduce_32<T>(vals, lane);
      if ((lane & 1) == 0) s_wave[wave][NB + ((lane >> 1) & 31)] = total;
      if (live && r == j + 1) {
#pragma unroll
        for (int k = 0; k < NB; ++k) s_piv_out[NB + k] = a[k];
      }
    }
    __syncthreads();
    if (tid < width) {
      const T sum = (s_wave[0][tid] + s_wave[1][tid]) + (s_wave[2][tid] + s_wave[3][tid]);
      __hip_atomic_store(part_c + wg * 2 * NB + tid, mailbox_pack(sum, seq), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const int pivot_row = tid < NB ? j : j + 1;
      if (pivot_row >= p + wg * 256 && pivot_row < p + wg * 256 + 256)  // this workgroup owns that pivot row
        __hip_atomic_store(piv_c + tid, mailbox_pack(s_piv_out[tid], seq), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    {
      // fixed-order sums of the per-workgroup partials: thread (k, g) takes value k of the workgroups
      // g, g + 4, ..., sixteen loads in flight
      const int k = tid & (2 * NB - 1), g = tid >> 6;
      T s = T(0);
      bool ok = true;
      if (k < width) {
        for (int w0 = g; w0 < nwg && ok; w0 += 64) {
          const unsigned long long* slot[16];
          bool used[16];
          float v[16];
#pragma unroll
          for (int u = 0; u < 16; ++u) {
            used[u] = w0 + 4 * u < nwg;
            slot[u] = part_c + (used[u] ? (w0 + 4 * u) : 0) * 2 * NB + k;
          }
          ok = mailbox_wait<16>(slot, used, seq, error, spin_limit, v);
#pragma unroll
          for (int u = 0; u < 16; ++u) s += v[u];
        }
      }
      s_sum4[g][k] = s;
      if (tid < width && ok) {
        const unsigned long long* slot[1] = {piv_c + tid};
        const bool used[1] = {true};
        float v[1];
        ok = mailbox_wait<1>(slot, used, seq, error, spin_limit, v);
        s_piv[tid] = v[0];
      }
      if (!ok) {
        __hip_atomic_store(error, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_fail = 1;
      }
    }
    __syncthreads();
    if (s_fail) return;
    if (tid < width) s_tot[tid] = (s_sum4[0][tid] + s_sum4[1][tid]) + (s_sum4[2][tid] + s_sum4[3][tid]);
    __syncthreads();
    if (tid < NB) {
      const int k = tid;
      const T seen = s_scal[6];  // largest squared column norm of this panel so far (0 at its first column)
      const Reflector h0 = make_reflector(s_piv[0], s_tot[0], kQrNegligible * seen);
      T seen_next = fmaxf(seen, s_piv[0] * s_piv[0] + s_tot[0]);
      const T tc0 = (k >= 1) ? h0.tau * (s_piv[k] + h0.scale * s_tot[k]) : T(0);
      s_tc[0][k] = tc0;
      if (k == 0) {
        s_scal[0] = h0.scale; s_scal[1] = h0.beta; s_scal[2] = h0.tau;
      }
      T seen_out = seen_next;
      if (pair) {
        // row j+1 and the sums over the rows below it, after reflector j
        const T q0 = s_piv[NB];                              // a_0[j+1]
        const T v0_next = h0.scale * q0;                     // v[j+1]
        const T tc0_1 = h0.tau * (s_piv[1] + h0.scale * s_tot[1]);
        const T piv1 = s_piv[NB + k] - tc0 * v0_next;        // a'_k[j+1], k >= 1
        const T sp_k = s_tot[k] - q0 * s_piv[NB + k];        // <a_0, a_k> below row j+1
        const T sp_0 = s_tot[0] - q0 * q0;
        const T sp_1 = s_tot[1] - q0 * s_piv[NB + 1];
        const T u_k = s_tot[NB + k] - tc0 * h0.scale * sp_1 - tc0_1 * h0.scale * sp_k +
                      tc0_1 * tc0 * h0.scale * h0.scale * sp_0;
        // lane 1 holds the corrected squared norm of column j+1 below its pivot and its pivot entry
        // (the last column of the matrix has nothing below its pivot: exactly zero, so tau = 0 as in LAPACK)
        const T x2_1 = (j + 1 < n - 1) ? __shfl(u_k, 1, 64) : T(0), alpha1 = __shfl(piv1, 1, 64);
        // size of the terms the corrected norm is the difference of (all three are >= 0 in exact arithmetic)
        const T magnitude = s_tot[NB + 1] + T(2) * fabsf(tc0_1 * h0.scale * sp_1) +
                            tc0_1 * tc0_1 * h0.scale * h0.scale * fabsf(sp_0);
        const bool ok = (x2_1 - x2_1 == T(0)) && x2_1 >= kQrPairGuard * magnitude;  // finite and no cancellation
        const Reflector h1 = make_reflector(alpha1, fmaxf(x2_1, T(0)), kQrNegligible * seen_next);
        if (ok) seen_next = fmaxf(seen_next, alpha1 * alpha1 + fmaxf(x2_1, T(0)));
        s_tc[1][k] = (k >= 2) ? h1.tau * (piv1 + h1.scale * u_k) : T(0);
        seen_out = seen_next;
        if (k == 0) {
          s_scal[3] = h1.scale; s_scal[4] = h1.beta; s_scal[5] = h1.tau;
          s_pair_ok = ok ? 1 : 0;
        }
      } else if (k == 0) {
        s_pair_ok = 0;
      }
      // every lane read s_scal[6] above; lane 0 of the same wavefront may now replace it
      if (k == 0) s_scal[6] = seen_out;
    }
    __syncthreads();
    const bool two = s_pair_ok != 0;
    {
      const T scale = s_scal[0], beta = s_scal[1], tauv = s_scal[2];
      if (live && r >= j) {
        if (r > j) {
          const T v = a[0] * scale;
          a[0] = v;
#pragma unroll
          for (int k = 1; k < NB; ++k) a[k] -= s_tc[0][k] * v;
        } else {
          a[0] = beta;
#pragma unroll
          for (int k = 1; k < NB; ++k) a[k] -= s_tc[0][k];
          tau[j] = tauv;
        }
      }
      if (live) {
        A[r + (int64_t)j * lda] = a[0];  // column j is final
        vout[(r - vrow0) + (int64_t)c * ldv] = (r > j) ? a[0] : (r == j ? T(1) : T(0));
      }
    }
    if (two) {
      const T scale = s_scal[3], beta = s_scal[4], tauv = s_scal[5];
      const int j1 = j + 1;
      if (live && r >= j1) {
        if (r > j1) {
          const T v = a[1] * scale;
          a[1] = v;
#pragma unroll
          for (int k = 2; k < NB; ++k) a[k] -= s_tc[1][k] * v;
        } else {
          a[1] = beta;
#pragma unroll
          for (int k = 2; k < NB; ++k) a[k] -= s_tc[1][k];
          tau[j1] = tauv;
        }
      }
      if (live) {
        A[r + (int64_t)j1 * lda] = a[1];
        vout[(r - vrow0) + (int64_t)(c + 1) * ldv] = (r > j1) ? a[1] : (r == j1 ? T(1) : T(0));
      }
#pragma unroll
      for (int k = 0; k + 2 < NB; ++k) a[k] = a[k + 2];
      a[NB - 2] = T(0);
      a[NB - 1] = T(0);
      c += 2;
    } else {
#pragma unroll
      for (int k = 0; k + 1 < NB; ++k) a[k] = a[k + 1];
      a[NB - 1] = T(0);
      c += 1;
    }
    // No barrier here: the shared arrays of the next round's first phase (s_wave, s_piv_out) were
    // last read before the barrier that follows the mailbox phase, and the arrays read above are
    // rewritten only behind the next such barrier, which every wavefront reaches after this point.
  }
}

// Vc (nrows x nbw, ld ldv) <- the unit-lower-trapezoidal reflector block stored in A with its
// unit diagonal at (row0 + c, col0 + c): zeros above, ones on, A below.
template <typename T>
__global__ void extract_v_kernel(const T* __restrict__ A, int64_t lda, int nrows, int row0, int col0, int nbw,
                                 T* __restrict__ Vc, int64_t ldv) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;  // row within the block
  if (i >= nrows) return;
  for (int c = blockIdx.y; c < nbw; c += gridDim.y) {
    T v;
    if (i < c) v = T(0);
    else if (i == c) v = T(1);
    else v = A[(row0 + i) + (int64_t)(col0 + c) * lda];
    Vc[i + (int64_t)c * ldv] = v;
  }
}

// Value of `v` in lane `LANE` (a compile-time constant) as a wavefront-uniform scalar.
template <int LANE>
__device__ __forceinline__ float lane_value(float v) {
  return __uint_as_float((unsigned)__builtin_amdgcn_readlane((int)__float_as_uint(v), LANE));
}
template <int LANE>
__device__ __forceinline__ double lane_value(double v) {
  const int lo = __builtin_amdgcn_readlane(__double2loint(v), LANE);
  const int hi = __builtin_amdgcn_readlane(__double2hiint(v), LANE);
  return __hiloint2double(hi, lo);
}

// Column I of the factor, for I = 0 .. 31 by recursion: lane k holds row k of T in t[] and row k of
// G in g[]; T[0:I, I] = -tau_I T[0:I, 0:I] G[0:I, I], where G[l, I] is fetched from lane l's
// register and T[k, l] is zero below the diagonal, so every lane runs the same I multiply-adds.
template <typename T, int I>
struct LarftColumn {
  template <int L>
  static __device__ __forceinline__ T dot(const T (&t)[32], const T& g_i) {
    if constexpr (L < 0) {
      return T(0);
    } else {
      return dot<L - 1>(t, g_i) + t[L] * lane_value<L>(g_i);
    }
  }
  static __device__ __forceinline__ void run(T (&t)[32], const T (&g)[32], T tau_k, int k) {
    if constexpr (I > 0) LarftColumn<T, I - 1>::run(t, g, tau_k, k);
    const T tau_i = lane_value<I>(tau_k);
    const T acc = dot<I - 1>(t, g[I]);
    t[I] = (k < I) ? -tau_i * acc : (k == I ? tau_i : T(0));
  }
};

// Compact-WY factor of up to 32 reflectors: T upper triangular with H_0 ... H_{w-1} = I - V T V^T,
// from G = V^T V (LAPACK larft, forward / columnwise).  One wavefront per 32-wide diagonal block:
// blockIdx.x selects the block (G, tau and T advance along the diagonal), so the diagonal blocks
// of a wider factor are built by one launch.  Everything stays in registers: the recursion over
// the columns is unrolled at compile time and values cross lanes as scalars (v_readlane).
// Reflectors beyond the block's width count as tau = 0, which leaves their rows and columns zero.
// G may arrive as `splits` unreduced split-K slices (`slab` elements apart), summed while loading.
template <typename T>
__global__ __launch_bounds__(128) void larft32_kernel(const T* __restrict__ G, int ldg, int splits, int64_t slab,
                                                       const T* __restrict__ tau, int nbw, T* __restrict__ Tm,
                                                       int ldt) {
  __shared__ T s_g[4][32][33];
  const int b = blockIdx.x;
  const int w = min(32, nbw - 32 * b);
  G += (int64_t)32 * b * (ldg + 1);
  Tm += (int64_t)32 * b * (ldt + 1);
  tau += 32 * b;
  const int k = threadIdx.x & 31, zg = threadIdx.x >> 5;
  T t[32], g[32];
  // slices z = zg, zg + 4, ... are summed by slice group zg (128 threads = 4 groups), the groups then
  // in a fixed order
#pragma unroll
  for (int c = 0; c < 32; ++c) g[c] = T(0);
  if (k < w) {
    for (int z = zg; z < splits; z += 4) {
      const T* slice = G + (int64_t)z * slab + k;
#pragma unroll
      for (int c = 0; c < 32; ++c) g[c] += (c < w) ? slice[c * ldg] : T(0);
    }
  }
  if (splits > 1) {
#pragma unroll
    for (int c = 0; c < 32; ++c) s_g[zg][k][c] = g[c];
    __syncthreads();
    if (zg == 0) {
#pragma unroll
      for (int c = 0; c < 32; ++c)
        g[c] = (s_g[0][k][c] + s_g[1][k][c]) + (s_g[2][k][c] + s_g[3][k][c]);
    }
  }
  if (threadIdx.x >= 64) return;  // the recursion runs in the first wavefront; its lanes 32..63 carry zeros
  const int lane = threadIdx.x;
  if (lane >= 32) {
#pragma unroll
    for (int c = 0; c < 32; ++c) g[c] = T(0);
  }
#pragma unroll
  for (int c = 0; c < 32; ++c) t[c] = T(0);
  const T tau_k = (lane < w) ? tau[lane] : T(0);
  LarftColumn<T, 31>::run(t, g, tau_k, lane);
  if (lane < w) {
#pragma unroll
    for (int c = 0; c < 32; ++c)
      if (c < w) Tm[lane + c * ldt] = t[c];
  }
}

// Fills the diagonal of Q with NaN if the error flag is set.
template <typename T>
__global__ void poison_on_error_kernel(T* __restrict__ Q, int64_t ldq, int n, const int* __restrict__ error) {
  if (*error == 0) return;
  for (int i = threadIdx.x; i < n; i += blockDim.x) Q[i + (int64_t)i * ldq] = T(NAN);
}

template <typename T>
__global__ void fill_zero_kernel(T* __restrict__ p, int count) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) p[i] = T(0);
}

// Finishes the block columns [p, p + nbw) of the explicit Q: rows above the block are zero and the
// unit diagonal of [I; 0] is added to -V (T V1^T).
template <typename T>
__global__ void orgqr_panel_fix_kernel(T* __restrict__ Q, int64_t ldq, int p, int nbw) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < p) {
    for (int c = 0; c < nbw; ++c) Q[i + (int64_t)(p + c) * ldq] = T(0);
  } else if (i < p + nbw) {
    Q[i + (int64_t)i * ldq] += T(1);
  }
}

// ---- block reflectors ------------------------------------------------------------------------
constexpr int kBrMax = 256;   // widest block reflector (outer block of the QR, back-transformation)
constexpr int kBrSplits = 8;  // split-K slices of the tall-skinny products

template <typename T>
struct BlockReflectorWs {
  T* v;       // n x kBrMax   clean reflector block
  T* gram;    // kBrMax x kBrMax
  T* w;       // kBrMax x n
  T* w2;      // kBrMax x n
  T* mx;      // kBrMax x kBrMax
  T* splitk;  // kBrSplits x kBrMax x n
};

template <typename T, class WS>
static inline void block_reflector_layout(WS& ws, int64_t n, BlockReflectorWs<T>* out) {
  BlockReflectorWs<T> b;
  b.v = ws.template take<T>((size_t)n * kBrMax);
  b.gram = ws.template take<T>(kBrMax * kBrMax);
  b.w = ws.template take<T>((size_t)n * kBrMax);
  b.w2 = ws.template take<T>((size_t)n * kBrMax);
  b.mx = ws.template take<T>(kBrMax * kBrMax);
  b.splitk = ws.template take<T>((size_t)kBrSplits * kBrMax * n);
  if (out) *out = b;
}

// T (ld kBrMax) from G = V^T V (in ws.gram, ld kBrMax) and tau for nbw <= kBrMax reflectors.  The
// diagonal 32-blocks [first_block, ...) come from larft32_kernel (earlier ones are already in Tm,
// the rest of Tm must be zero); block column j then follows from the blocks to its left:
//   T[0:R, j] = -T[0:R, 0:R] (G[0:R, j] T[j, j]),  R = 32 j.
template <typename T>
static inline int assemble_t_factor(hipStream_t s, const BlockReflectorWs<T>& ws, int nbw, const T* tau, T* Tm,
                                    int first_block) {
  using Skinny = typename SkinnyTile<T>::type;
  const int blocks = (int)ceil_div64(nbw, 32);
  if (first_block < blocks) {
    hipLaunchKernelGGL((larft32_kernel<T>), dim3(blocks - first_block), dim3(128), 0, s,
                       ws.gram + (int64_t)32 * first_block * (kBrMax + 1), kBrMax, 1, (int64_t)0, tau + 32 * first_block,
                       nbw - 32 * first_block, Tm + (int64_t)32 * first_block * (kBrMax + 1), kBrMax);
    SOAPMI_LAUNCH_CHECK();
  }
  for (int j = 1; j < blocks; ++j) {
    const int R = 32 * j, wj = std::min(32, nbw - R);
    int rc = gemm<T, Skinny>(s, 0, 0, R, wj, wj, T(1), ws.gram + (int64_t)R * kBrMax, kBrMax,
                             Tm + (int64_t)R * (kBrMax + 1), kBrMax, T(0), ws.mx, kBrMax);
    if (rc) return rc;
    rc = gemm<T, Skinny>(s, 0, 0, R, wj, R, T(-1), Tm, kBrMax, ws.mx, kBrMax, T(0), Tm + (int64_t)R * kBrMax, kBrMax);
    if (rc) return rc;
  }
  return kOk;
}

// Number of K slices for a tall-skinny product with `tiles` output tiles, K = rows, an M x N
// output: enough slices to occupy the chip (about 512 workgroups), at least 128 rows each, and no
// more partial results than the split-K buffer (kBrSplits * kBrMax * ldv elements) holds.
static inline int split_count(int64_t tiles, int rows, int M, int N, int64_t ldv) {
  if (rows < 512) return 1;
  int64_t splits = std::min<int64_t>(ceil_div64(512, tiles), rows / 128);
  const int64_t capacity = (int64_t)kBrSplits * kBrMax * ldv / std::max<int64_t>(1, (int64_t)M * N);
  splits = std::min<int64_t>(splits, std::min<int64_t>(capacity, 64));
  return (int)std::max<int64_t>(splits, 1);
}

// W2 (M x N, ld ldw2) = op(T) * (sum of the split-K slices of W), M <= 32: the middle product of a
// 32-wide block reflector, taking V^T C straight from the slices (slice z at part + z * slab,
// leading dimension M).  256 threads own 32 rows x 2 columns x 4 groups of slices.
template <typename T>
__global__ __launch_bounds__(256) void reflector_w2_kernel(const T* __restrict__ part, int splits, int64_t slab, int M,
                                                           int N, const T* __restrict__ Tm, int ldt, int trans_t,
                                                           T* __restrict__ W2, int ldw2) {
  __shared__ T s_t[32][33];
  __shared__ T s_w[2][4][33];
  const int tid = threadIdx.x, l = tid & 31, zg = (tid >> 5) & 3, cc = tid >> 7;
  const int c = blockIdx.x * 2 + cc;
  for (int q = tid >> 5; q < 32; q += 8) {  // s_t[a][b] = op(T)[a, b]
    const T v = (l < M && q < M) ? Tm[l + q * ldt] : T(0);  // T[l, q]
    if (trans_t) s_t[q][l] = v;
    else s_t[l][q] = v;
  }
  T sum = T(0);
  if (l < M && c < N)
    for (int z = zg; z < splits; z += 4) sum += part[(int64_t)z * slab + l + (int64_t)c * M];
  s_w[cc][zg][l] = sum;
  __syncthreads();
  if (zg == 0 && l < M && c < N) {
    T acc = T(0);
#pragma unroll
    for (int q = 0; q < 32; ++q)
      acc += s_t[l][q] * ((s_w[cc][0][q] + s_w[cc][1][q]) + (s_w[cc][2][q] + s_w[cc][3][q]));
    W2[l + (int64_t)c * ldw2] = acc;
  }
}

template <typename T>
static inline int gram_of_v(hipStream_t s, const BlockReflectorWs<T>& ws, int rows, int nbw, int64_t ldv) {
  using Skinny = typename SkinnyTile<T>::type;
  const int splits = split_count(1, rows, nbw, nbw, ldv);
  if (nbw <= Skinny::BM)
    return gemm<T, Skinny>(s, 1, 0, nbw, nbw, rows, T(1), ws.v, ldv, ws.v, ldv, T(0), ws.gram, kBrMax, splits,
                           ws.splitk);
  return gemm<T>(s, 1, 0, nbw, nbw, rows, T(1), ws.v, ldv, ws.v, ldv, T(0), ws.gram, kBrMax, splits, ws.splitk);
}

// V (rows x nbw, in ws.v, ld ldv) is in place; computes T (ld kBrMax, fully overwritten) from
// V^T V and tau.
template <typename T>
static inline int build_t_factor(hipStream_t s, const BlockReflectorWs<T>& ws, int rows, int nbw, int64_t ldv,
                                 const T* tau, T* Tm) {
  hipLaunchKernelGGL((fill_zero_kernel<T>), dim3(kBrMax * kBrMax / 256), dim3(256), 0, s, Tm, kBrMax * kBrMax);
  int rc = gram_of_v<T>(s, ws, rows, nbw, ldv);
  if (rc) return rc;
  return assemble_t_factor<T>(s, ws, nbw, tau, Tm, 0);
}

// C (rows x nc, ld ldc) <- C - V op(T) V^T C.
template <typename T>
static inline int apply_block_reflector(hipStream_t s, const BlockReflectorWs<T>& ws, const T* Tm, bool transT,
                                        int rows, int nbw, int nc, int64_t ldv, T* C, int64_t ldc) {
  using Skinny = typename SkinnyTile<T>::type;
  using Wide = typename DefaultTile<T>::type;
  if (nc <= 0 || rows <= 0 || nbw <= 0) return kOk;
  const bool skinny = nbw <= Skinny::BM;
  // W = V^T C  (nbw x nc, K = rows): few output tiles, long K -> split-K with a fixed-order reduce
  const int64_t tiles = ceil_div64(nc, skinny ? Skinny::BN : Wide::BN) * ceil_div64(nbw, skinny ? Skinny::BM : Wide::BM);
  const int splits = split_count(tiles, rows, nbw, nc, ldv);
  int rc;
  if (skinny) {
    int slices = 1;
    rc = gemm_to_partials<T, Skinny>(s, 1, 0, nbw, nc, rows, ws.v, ldv, C, ldc, splits, ws.splitk, &slices);
    if (rc) return rc;
    hipLaunchKernelGGL((reflector_w2_kernel<T>), dim3((unsigned)ceil_div64(nc, 2)), dim3(256), 0, s, ws.splitk, slices,
                       (int64_t)nbw * nc, nbw, nc, Tm, kBrMax, transT ? 1 : 0, ws.w2, kBrMax);
    SOAPMI_LAUNCH_CHECK();
    rc = kOk;
  } else {
    rc = gemm<T>(s, 1, 0, nbw, nc, rows, T(1), ws.v, ldv, C, ldc, T(0), ws.w, kBrMax, splits, ws.splitk);
    if (rc) return rc;
    rc = gemm<T>(s, transT ? 1 : 0, 0, nbw, nc, nbw, T(1), Tm, kBrMax, ws.w, kBrMax, T(0), ws.w2, kBrMax);
  }
  if (rc) return rc;
  // C -= V W2
  return gemm<T>(s, 0, 0, rows, nc, nbw, T(-1), ws.v, ldv, ws.w2, kBrMax, T(1), C, ldc);
}

template <typename T>
static inline void launch_extract_v(hipStream_t s, const T* A, int64_t lda, int rows, int row0, int col0, int nbw,
                                    T* V, int64_t ldv) {
  hipLaunchKernelGGL((extract_v_kernel<T>), dim3((unsigned)ceil_div64(rows, 256), (unsigned)std::min(nbw, 32)),
                     dim3(256), 0, s, A, lda, rows, row0, col0, nbw, V, ldv);
}

// ---- QR driver -------------------------------------------------------------------------------
template <typename T>
struct QrWorkspace {
  BlockReflectorWs<T> br;
  T* t_all;   // outer blocks x kBrMax x kBrMax
  T* tau;     // n
  T* part;    // 2 x nwg x NB   partials of the launch-per-column fallback
  T* piv;     // 2 x NB
  unsigned long long* mail_part;  // 2 x kQrPersistentMaxWg x 2 NB   mailboxes of the persistent panel kernel
  unsigned long long* mail_piv;   // 2 x 2 NB
  unsigned* sync;  // [1] error flag of the persistent panel kernel
};

template <typename T, class WS>
static inline void qr_workspace_layout(WS& ws, int64_t n, QrWorkspace<T>* out) {
  QrWorkspace<T> q;
  const int64_t blocks = ceil_div64(n, kBrMax);
  const int64_t nwg = ceil_div64(n, 256);
  block_reflector_layout<T>(ws, n, out ? &q.br : nullptr);
  q.t_all = ws.template take<T>((size_t)blocks * kBrMax * kBrMax);
  q.tau = ws.template take<T>((size_t)n);
  q.part = ws.template take<T>((size_t)2 * nwg * kQrNb);
  q.piv = ws.template take<T>(2 * kQrNb);
  q.mail_part = ws.template take<unsigned long long>((size_t)2 * kQrPersistentMaxWg * 2 * kQrNb);
  q.mail_piv = ws.template take<unsigned long long>(2 * 2 * kQrNb);
  q.sync = ws.template take<unsigned>(64);
  if (out) *out = q;
}

template <typename T>
static inline size_t qr_workspace_bytes(int64_t n) {
  WorkspaceSizer sizer;
  qr_workspace_layout<T>(sizer, n, nullptr);
  return sizer.total();
}

// geqrf in place on A (n x n), then the explicit Q into Qout (n x n).  A is destroyed.
// Two levels of blocking: 32-column panels (register-resident column steps) are applied only
// inside their kBrMax-column outer block; the trailing matrix and Q see kBrMax-wide block
// reflectors, whose products have K = kBrMax and run on the full-size MFMA tile.
template <typename T>
static inline int qr_factor_and_form_q(hipStream_t s, T* A, int64_t lda, T* Qout, int64_t ldq, int n,
                                       const QrWorkspace<T>& ws, int persistent_max_wg = kQrPersistentMaxWg,
                                       unsigned spin_limit = kQrSpinLimit, int columns_per_round = 2) {
  const int NB = kQrNb, OB = kBrMax;
  const int blocks = (int)ceil_div64(n, OB);
  const int64_t ldv = n;
  int rc;
  static_assert(std::is_same<T, float>::value, "the persistent panel kernel packs float values into its mailboxes");
  unsigned seq_base = 0;
  hipLaunchKernelGGL((fill_zero_kernel<unsigned>), dim3(1), dim3(64), 0, s, ws.sync, 64);
  {
    // mail_part and mail_piv are adjacent: one clear covers both (sequence number 0 = "nothing yet")
    const int words = 2 * (2 * kQrPersistentMaxWg * 2 * kQrNb + 2 * 2 * kQrNb);
    hipLaunchKernelGGL((fill_zero_kernel<unsigned>), dim3((words + 255) / 256), dim3(256), 0, s,
                       reinterpret_cast<unsigned*>(ws.mail_part), words);
  }
  // ---- factorisation ----
  for (int bi = 0; bi < blocks; ++bi) {
    const int P = bi * OB, PE = std::min(n, P + OB), obw = PE - P;
    T* Tm = ws.t_all + (size_t)bi * OB * OB;
    hipLaunchKernelGGL((fill_zero_kernel<T>), dim3(OB * OB / 256), dim3(256), 0, s, Tm, OB * OB);
    int inner_done = 0;
    bool v_written = true;  // the panel kernels leave the block's reflectors in ws.br.v
    for (int p = P; p < PE; p += NB) {
      const int pe = std::min(PE, p + NB), nbw = pe - p;
      const int rows = n - p;
      const int nwg = (int)ceil_div64(rows, 256);
      T* part[2] = {ws.part, ws.part + (size_t)nwg * NB};
      T* piv[2] = {ws.piv, ws.piv + NB};
      // this panel's reflectors inside the outer block's n x 128 buffer (origin: row P, column P)
      BlockReflectorWs<T> inner = ws.br;
      inner.v = ws.br.v + (p - P) + (int64_t)(p - P) * ldv;
      if (nwg <= persistent_max_wg) {
        hipLaunchKernelGGL(qr_panel_persistent_kernel, dim3(nwg), dim3(256), 0, s, A, lda, n, p, pe, ws.mail_part,
                           ws.mail_piv, ws.tau, seq_base, reinterpret_cast<int*>(ws.sync + 1), nwg, spin_limit,
                           ws.br.v + (int64_t)(p - P) * ldv, ldv, P, columns_per_round >= 2 ? 1 : 0);
        seq_base += (unsigned)nbw;
      } else {
        for (int j = p - 1; j < pe; ++j) {
          const int in = (j - p + 1) & 1, out = in ^ 1;
          hipLaunchKernelGGL((qr_panel_step_kernel<T>), dim3(nwg), dim3(256), 0, s, A, lda, n, p, pe, j, part[in],
                             piv[in], part[out], piv[out], ws.tau, nwg);
        }
        v_written = false;
      }
      SOAPMI_LAUNCH_CHECK();
      if (pe < PE) {  // the panel's reflectors act on the rest of the outer block only
        T* Tin = Tm + (int64_t)(p - P) * (OB + 1);  // diagonal block of the outer factor
        if (!v_written) launch_extract_v<T>(s, A, lda, rows, p, p, nbw, inner.v, ldv);
        int slices = 1;  // V^T V stays in split-K slices; the factor kernel sums them while loading
        rc = gemm_to_partials<T, typename SkinnyTile<T>::type>(s, 1, 0, nbw, nbw, rows, inner.v, ldv, inner.v, ldv,
                                                               split_count(1, rows, nbw, nbw, ldv), inner.splitk,
                                                               &slices);
        if (rc) return rc;
        hipLaunchKernelGGL((larft32_kernel<T>), dim3(1), dim3(128), 0, s, inner.splitk, nbw, slices,
                           (int64_t)nbw * nbw, ws.tau + p, nbw, Tin, OB);
        SOAPMI_LAUNCH_CHECK();
        rc = apply_block_reflector<T>(s, inner, Tin, true, rows, nbw, PE - pe, ldv, A + p + (int64_t)pe * lda, lda);
        if (rc) return rc;
        ++inner_done;
      }
    }
    const int rows = n - P;
    if (!v_written) launch_extract_v<T>(s, A, lda, rows, P, P, obw, ws.br.v, ldv);
    rc = gram_of_v<T>(s, ws.br, rows, obw, ldv);
    if (rc) return rc;
    rc = assemble_t_factor<T>(s, ws.br, obw, ws.tau + P, Tm, inner_done);
    if (rc) return rc;
    // trailing columns: C <- H^T C = C - V T^T V^T C
    rc = apply_block_reflector<T>(s, ws.br, Tm, true, rows, obw, n - PE, ldv, A + P + (int64_t)PE * lda, lda);
    if (rc) return rc;
  }
  // ---- explicit Q, outer blocks in reverse ----
  for (int bi = blocks - 1; bi >= 0; --bi) {
    const int P = bi * OB, PE = std::min(n, P + OB), obw = PE - P;
    const int rows = n - P;
    T* Tm = ws.t_all + (size_t)bi * OB * OB;
    launch_extract_v<T>(s, A, lda, rows, P, P, obw, ws.br.v, ldv);
    SOAPMI_LAUNCH_CHECK();
    // columns to the right already hold Q of the later blocks: C <- (I - V T V^T) C
    rc = apply_block_reflector<T>(s, ws.br, Tm, false, rows, obw, n - PE, ldv, Qout + P + (int64_t)PE * ldq, ldq);
    if (rc) return rc;
    // own columns: [I;0] - V (T V1^T)
    rc = gemm<T>(s, 0, 1, obw, obw, obw, T(1), Tm, OB, ws.br.v, ldv, T(0), ws.br.mx, OB);
    if (rc) return rc;
    rc = gemm<T>(s, 0, 0, rows, obw, obw, T(-1), ws.br.v, ldv, ws.br.mx, OB, T(0), Qout + P + (int64_t)P * ldq, ldq);
    if (rc) return rc;
    hipLaunchKernelGGL((orgqr_panel_fix_kernel<T>), dim3((unsigned)ceil_div64(PE, 256)), dim3(256), 0, s, Qout, ldq, P,
                       obw);
    SOAPMI_LAUNCH_CHECK();
  }
  // A panel kernel that gave up waiting leaves garbage behind: make that impossible to miss.
  hipLaunchKernelGGL((poison_on_error_kernel<T>), dim3(1), dim3(64), 0, s, Qout, ldq, n,
                     reinterpret_cast<const int*>(ws.sync + 1));
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

}  // namespace soapmi
