// Blocked Householder QR (LAPACK geqrf sign convention) and explicit formation of Q, for the
// power-iteration refresh of a SOAP eigenbasis (what the reference obtains from SLATE's
// geqrf + unmqr on the identity: src/soap_tp/csrc/slate_bindings.cpp:176-185).
//
// Panel (NB = 32 columns): a workgroup owns 256 rows, one per thread, and keeps its row of the
// panel in registers.  Normally the whole panel runs in one persistent launch whose workgroups
// exchange, once, the 32 x 32 Gram matrix of their rows (computed on the matrix cores) through
// device memory; every workgroup then runs the panel's Householder steps on [top block ; Gram],
// applies the reflectors to its rows and leaves its slice of V^T [V | C] for the update of the
// rest of the outer block (qr_panel_gram_kernel).  qr_panel_persistent_kernel is the same launch
// with one to four columns per exchange and partial dot products instead of a Gram matrix; beyond
// kQrPersistentMaxWg workgroups the panel runs one launch per column (qr_panel_step_kernel: launch
// j applies reflector j, whose dot products with the remaining panel columns were reduced by launch
// j-1, and in the same pass reduces the dot products reflector j+1 needs).  Sums over workgroups
// have a fixed order and use no atomics on data, so results do not depend on scheduling.
// In-block update: one launch per panel (panel_apply_kernel).  Trailing matrix and Q formation:
// compact-WY block reflectors on the MFMA GEMM.
#pragma once
#include <type_traits>
#include <vector>

#include "common.hpp"
#include "gemm.hpp"

namespace soapmi {

constexpr int kQrNb = 32;

// 32 values per lane are summed over the wavefront by a butterfly: at every stage a lane keeps one
// half of its values (which half is decided by one bit of its lane number), sends the other half to
// a partner lane and adds what the partner sends for the half it keeps.
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

// The narrow stages on data-parallel-primitive moves (no trip through the LDS crossbar): the
// partner is lane ^ 15 (row_mirror), lane ^ 7 (row_half_mirror), lane ^ 2 and lane ^ 1 (quad_perm).
// Together with the two swap stages (lane ^ 32, lane ^ 16) these six masks reach every lane of the
// wavefront, and which half a lane keeps at a stage is decided by one bit of its own number, so the
// value index a lane ends up with is the same as with the plain xor pattern.
template <int CTRL>
__device__ __forceinline__ float dpp_partner(float v) {
  return __uint_as_float((unsigned)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), CTRL, 0xF, 0xF, false));
}
template <int CTRL>
__device__ __forceinline__ double dpp_partner(double v) {
  const int lo = __builtin_amdgcn_update_dpp(0, __double2loint(v), CTRL, 0xF, 0xF, false);
  const int hi = __builtin_amdgcn_update_dpp(0, __double2hiint(v), CTRL, 0xF, 0xF, false);
  return __hiloint2double(hi, lo);
}

constexpr int kDppRowMirror = 0x140, kDppRowHalfMirror = 0x141, kDppQuadXor2 = 0x4E, kDppQuadXor1 = 0xB1;

template <typename T, int HALF, int BIT, int CTRL>
__device__ __forceinline__ void butterfly_stage_dpp(T (&vals)[32], int lane) {
  const bool upper = (lane & BIT) != 0;
#pragma unroll
  for (int c = 0; c < HALF; ++c) {
    const T send = upper ? vals[c] : vals[c + HALF];
    const T keep = upper ? vals[c + HALF] : vals[c];
    vals[c] = keep + dpp_partner<CTRL>(send);
  }
}

// After the call lane l holds, in the return value, the sum over the wavefront of vals[(l>>1)&31].
// Stages are spelled out so that every register index is a compile-time constant.
template <typename T>
__device__ __forceinline__ T wave_reduce_32(T (&vals)[32], int lane) {
  butterfly_stage_swap<T, 16, true>(vals);
  butterfly_stage_swap<T, 8, false>(vals);
  butterfly_stage_dpp<T, 4, 8, kDppRowMirror>(vals, lane);
  butterfly_stage_dpp<T, 2, 4, kDppRowHalfMirror>(vals, lane);
  butterfly_stage_dpp<T, 1, 2, kDppQuadXor2>(vals, lane);
  return vals[0] + dpp_partner<kDppQuadXor1>(vals[0]);
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

// Waits for and sums, in order, the words base[0], base[stride], ... of the first `count` of COUNT
// slots and likewise `count3` of EXTRA slots from base3 (every slot is loaded whether it counts or
// not, so all must be valid memory: the addresses are then constant offsets from two bases, which
// keeps this many loads in flight within the register budget).  False after too many polls or once
// the error flag is up.
template <int COUNT, int STRIDE, int EXTRA, int STRIDE3>
__device__ __forceinline__ bool mailbox_wait_sum(const unsigned long long* base, int count,
                                                 const unsigned long long* base3, int count3, unsigned seq,
                                                 const int* error, unsigned spin_limit, float& sum, float& sum3) {
  unsigned spins = 0;
  for (;;) {
    unsigned long long word[COUNT + EXTRA];
#pragma unroll
    for (int u = 0; u < COUNT; ++u)
      word[u] = __hip_atomic_load(base + u * STRIDE, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int u = 0; u < EXTRA; ++u)
      word[COUNT + u] = __hip_atomic_load(base3 + u * STRIDE3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    bool ready = true;
#pragma unroll
    for (int u = 0; u < COUNT; ++u) ready = ready && (u >= count || (unsigned)(word[u] >> 32) == seq);
#pragma unroll
    for (int u = 0; u < EXTRA; ++u) ready = ready && (u >= count3 || (unsigned)(word[COUNT + u] >> 32) == seq);
    if (ready) {
#pragma unroll
      for (int u = 0; u < COUNT; ++u) sum += (u < count) ? __uint_as_float((unsigned)word[u]) : 0.0f;
#pragma unroll
      for (int u = 0; u < EXTRA; ++u) sum3 += (u < count3) ? __uint_as_float((unsigned)word[COUNT + u]) : 0.0f;
      return true;
    }
    ++spins;
    if (spins > spin_limit) return false;
    if ((spins & 63u) == 0 && __hip_atomic_load(error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) return false;
    __builtin_amdgcn_s_sleep(1);
  }
}

// Everything a thread of the whole-panel kernel needs from an exchange, in one trip to memory, for
// launches of at most COUNT workgroups: its two Gram values from all workgroups (base0, base1,
// stride 64 words per workgroup), its share of the last sixteen values (base3, stride 16 x 64 words,
// `count3` <= EXTRA of them) and its four words of the top block.  The sums run over the workgroups
// in ascending order.  Every slot is loaded whether it counts or not.  False after too many polls
// or once the error flag is up.
template <int COUNT, int EXTRA>
__device__ __forceinline__ bool mailbox_wait_all(const unsigned long long* base0, const unsigned long long* base1,
                                                 int count, const unsigned long long* base3, int count3,
                                                 const unsigned long long* top, unsigned seq, const int* error,
                                                 unsigned spin_limit, float& sum0, float& sum1, float& sum3,
                                                 float (&top_value)[4]) {
  unsigned spins = 0;
  for (;;) {
    unsigned long long w0[COUNT], w1[COUNT], w3[EXTRA], wt[4];
#pragma unroll
    for (int u = 0; u < COUNT; ++u) w0[u] = __hip_atomic_load(base0 + u * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int u = 0; u < COUNT; ++u) w1[u] = __hip_atomic_load(base1 + u * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int u = 0; u < EXTRA; ++u)
      w3[u] = __hip_atomic_load(base3 + u * 16 * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int u = 0; u < 4; ++u) wt[u] = __hip_atomic_load(top + 256 * u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    bool ready = true;
#pragma unroll
    for (int u = 0; u < COUNT; ++u)
      ready = ready && (u >= count || ((unsigned)(w0[u] >> 32) == seq && (unsigned)(w1[u] >> 32) == seq));
#pragma unroll
    for (int u = 0; u < EXTRA; ++u) ready = ready && (u >= count3 || (unsigned)(w3[u] >> 32) == seq);
#pragma unroll
    for (int u = 0; u < 4; ++u) ready = ready && (unsigned)(wt[u] >> 32) == seq;
    if (ready) {
#pragma unroll
      for (int u = 0; u < COUNT; ++u) sum0 += (u < count) ? __uint_as_float((unsigned)w0[u]) : 0.0f;
#pragma unroll
      for (int u = 0; u < COUNT; ++u) sum1 += (u < count) ? __uint_as_float((unsigned)w1[u]) : 0.0f;
#pragma unroll
      for (int u = 0; u < EXTRA; ++u) sum3 += (u < count3) ? __uint_as_float((unsigned)w3[u]) : 0.0f;
#pragma unroll
      for (int u = 0; u < 4; ++u) top_value[u] = __uint_as_float((unsigned)wt[u]);
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

// The same scalars without a division or a correctly rounded square root on the critical path:
// with r = 1/sqrt(alpha^2 + x2) (hardware estimate plus one Newton step), tau = (beta - alpha)/beta
// = 1 + |alpha| r and scale = 1/(alpha - beta) = sign(alpha)/(|alpha| + norm) (reciprocal estimate
// plus one Newton step); each is within about one unit in the last place of the exact value.  Norms
// whose squares leave the comfortable part of the exponent range take the function above.
__device__ __forceinline__ Reflector make_reflector_fast(float alpha, float x2, float floor2) {
  const float nrm2 = alpha * alpha + x2;
  if (__builtin_expect(!(nrm2 > 1e-30f && nrm2 < 1e30f), 0)) return make_reflector(alpha, x2, floor2);
  const bool valid = x2 > 0.0f && nrm2 > floor2;
  float r = __builtin_amdgcn_rsqf(nrm2);
  r = r * (1.5f - 0.5f * nrm2 * r * r);
  const float nrm = nrm2 * r, absa = fabsf(alpha), den = absa + nrm;
  float inv = __builtin_amdgcn_rcpf(den);
  inv = inv * (2.0f - den * inv);
  Reflector h;
  h.beta = valid ? ((alpha >= 0.0f) ? -nrm : nrm) : alpha;
  h.tau = valid ? 1.0f + absa * r : 0.0f;
  h.scale = valid ? ((alpha >= 0.0f) ? inv : -inv) : 0.0f;
  return h;
}

// A column whose squared norm has fallen below kQrNegligible times the largest one met so far in
// its panel (a norm ratio of 1e-12) gets no reflector.  Such columns are rounding residue of
// exactly dependent columns; left to themselves they shrink by 1e-7 per column until their
// squares underflow, and a reflector built from underflowed sums is not orthogonal (LAPACK's
// slarfg rescales instead, which a norm that comes out of a reduction cannot do in place).
// What stays below the diagonal of R is below 1e-12 of the panel's scale; Q stays orthogonal.
constexpr float kQrNegligible = 1e-24f;

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

// Broadcast from one of the first kQrRoundMax lanes; `t` is a loop counter of a fully unrolled
// loop, so the switch folds to one v_readlane (a scalar broadcast instead of a trip through the
// LDS crossbar).
__device__ __forceinline__ float round_lane_value(float v, int t) {
  switch (t) {
    case 0: return lane_value<0>(v);
    case 1: return lane_value<1>(v);
    case 2: return lane_value<2>(v);
    default: return lane_value<3>(v);
  }
}

// a[k] <- a[k + D], zeros shifted in at the end; every index is a compile-time constant in range.
template <int D>
__device__ __forceinline__ void shift_left(float (&a)[kQrNb]) {
#pragma unroll
  for (int k = 0; k + D < kQrNb; ++k) a[k] = a[k + D];
#pragma unroll
  for (int k = kQrNb - D; k < kQrNb; ++k) a[k] = 0.0f;
}

// Several columns per message round.  A round covers the next `cols` <= kQrRoundMax panel columns
// j .. j+cols-1.  The workgroups exchange (a) the `cols` pivot rows j .. j+cols-1 in full and (b)
// the dot products G[t][k] = <a_t, a_k> of those columns with all remaining panel columns over the
// rows BELOW all the round's pivots.  With that, every workgroup runs the `cols` Householder steps
// on the compressed problem [pivot rows ; Gram of the rest]: the pivot rows are updated
// explicitly, and the dot products by the rank-one correction that applying reflector t to the
// hidden rows implies,
//   a_k <- a_k - tc_k s a_t   =>   G[i][k] <- G[i][k] - tc_k s G[i][t] - tc_i s G[t][k] + tc_i tc_k s^2 G[t][t]
// (s = the reflector's scale), so no further exchange is needed inside the round.  From the second
// step on a column's squared norm below its pivot is partly such a corrected number, a difference.
// Its terms' sizes are tracked alongside; when the norm falls below kQrRoundGuard times that size
// (cancellation: the column is nearly in the span of the round's earlier columns) the round ends
// before that step, the accepted reflectors are applied, and the column starts the next round, where
// its sums are computed directly.  Every workgroup takes these decisions from the same numbers in
// the same order.
constexpr int kQrRoundMax = 4;
constexpr float kQrRoundGuard = 0.25f;

__global__ __launch_bounds__(256) void qr_panel_persistent_kernel(float* __restrict__ A, int64_t lda, int n, int p,
                                                                  int pe, unsigned long long* part,
                                                                  unsigned long long* piv, float* __restrict__ tau,
                                                                  unsigned seq_base, int* error, int nwg,
                                                                  unsigned spin_limit, float* __restrict__ vout,
                                                                  int64_t ldv, int vrow0, int cols_cap) {
  using T = float;
  constexpr int NB = kQrNb, S = kQrRoundMax, W = S * NB;  // W values per workgroup and round at most
  __shared__ T s_wave[4][W];
  __shared__ T s_sum2[2][W];
  __shared__ T s_piv_out[W];
  __shared__ T s_tot[W];    // s_tot[t * NB + k] = G[t][k]
  __shared__ T s_piv[W];    // s_piv[t * NB + k] = entry k of pivot row j + t
  __shared__ T s_tc[S][NB];
  __shared__ T s_scal[S][3];  // scale, beta, tau of the round's reflectors
  __shared__ T s_seen;        // largest squared column norm of this panel so far
  __shared__ int s_accepted;
  __shared__ int s_fail;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wg = blockIdx.x;
  const int r = p + wg * 256 + tid;
  const int nbw = pe - p;
  const bool live = r < n;
  if (tid == 0) {
    s_fail = 0;
    s_seen = T(0);
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
    const int cols = min(min(cols_cap, S), nbw - c);
    const int width = cols * NB;  // values per workgroup in this round
    const unsigned seq = seq_base + round + 1u;
    unsigned long long* part_c = part + (size_t)(round & 1) * kQrPersistentMaxWg * W;
    unsigned long long* piv_c = piv + (round & 1) * W;
    // dot products of the round's columns with all panel columns over the rows below its pivots
    {
      const bool below = live && r > j + cols - 1;
#pragma unroll
      for (int t = 0; t < S; ++t) {
        if (t < cols) {
          T vals[NB];
#pragma unroll
          for (int k = 0; k < NB; ++k) vals[k] = below ? a[t] * a[k] : T(0);
          const T total = wave_reduce_32<T>(vals, lane);
          if ((lane & 1) == 0) s_wave[wave][t * NB + ((lane >> 1) & 31)] = total;
          if (live && r == j + t) {
#pragma unroll
            for (int k = 0; k < NB; ++k) s_piv_out[t * NB + k] = a[k];
          }
        }
      }
    }
    __syncthreads();
    if (tid < width) {
      const T sum = (s_wave[0][tid] + s_wave[1][tid]) + (s_wave[2][tid] + s_wave[3][tid]);
      __hip_atomic_store(part_c + wg * W + tid, mailbox_pack(sum, seq), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const int pivot_row = j + tid / NB;
      if (pivot_row >= p + wg * 256 && pivot_row < p + wg * 256 + 256)  // this workgroup owns that pivot row
        __hip_atomic_store(piv_c + tid, mailbox_pack(s_piv_out[tid], seq), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    {
      // fixed-order sums of the per-workgroup partials: thread (k, g) takes value k of the workgroups
      // g, g + 2, ..., up to thirty-two loads in flight
      const int k = tid & (W - 1), g = tid >> 7;
      T s = T(0);
      bool ok = true;
      if (k < width) {
        for (int w0 = g; w0 < nwg && ok; w0 += 64) {
          const unsigned long long* slot[32];
          bool used[32];
          float v[32];
#pragma unroll
          for (int u = 0; u < 32; ++u) {
            used[u] = w0 + 2 * u < nwg;
            slot[u] = part_c + (used[u] ? (w0 + 2 * u) : 0) * W + k;
          }
          ok = mailbox_wait<32>(slot, used, seq, error, spin_limit, v);
#pragma unroll
          for (int u = 0; u < 32; ++u) s += v[u];
        }
      }
      s_sum2[g][k] = s;
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
    if (tid < width) s_tot[tid] = s_sum2[0][tid] + s_sum2[1][tid];
    __syncthreads();
    if (tid < NB) {
      // Householder on the compressed problem; lane k owns column k of the pivot rows and of G
      const int k = tid;
      T pv[S], g[S];
#pragma unroll
      for (int t = 0; t < S; ++t) {
        pv[t] = (t < cols) ? s_piv[t * NB + k] : T(0);
        g[t] = (t < cols) ? s_tot[t * NB + k] : T(0);
      }
      // for lane k < cols: size of the terms G[k][k] is made of (its own value, then every correction)
      T size_diag = T(0);
#pragma unroll
      for (int t = 0; t < S; ++t)
        if (k == t) size_diag = fabsf(g[t]);
      T seen = s_seen;
      int accepted = 0;
#pragma unroll
      for (int t = 0; t < S; ++t) {
        if (t < cols && accepted == t) {
          // column t = lane t: leading entry pv[t], the explicit rows below it, and G[t][t]
          T explicit2 = T(0);
#pragma unroll
          for (int q = t + 1; q < S; ++q) explicit2 += pv[q] * pv[q];  // rows beyond `cols` hold zeros
          const T alpha = round_lane_value(pv[t], t);
          const T hidden2 = round_lane_value(g[t], t);
          const T x2_explicit = round_lane_value(explicit2, t);
          const T size_t_ = round_lane_value(size_diag, t);
          // (the last column of the matrix has nothing below its pivot: exactly zero, so tau = 0 as in LAPACK)
          const T x2 = (j + t < n - 1) ? x2_explicit + fmaxf(hidden2, T(0)) : T(0);
          // The reflector is orthogonal to the accuracy of alpha^2 + x2; alpha and the explicit rows are
          // exact, the hidden part carries an absolute error of about eps times the size of its terms.
          const bool finite = hidden2 - hidden2 == T(0);
          const bool ok = t == 0 || (finite && alpha * alpha + x2 >= kQrRoundGuard * size_t_);
          if (ok) {
            const Reflector h = make_reflector(alpha, x2, kQrNegligible * seen);
            seen = fmaxf(seen, alpha * alpha + x2);
            // d_k = <column t, column k> below pivot t
            T d = g[t];
#pragma unroll
            for (int q = t + 1; q < S; ++q) d += round_lane_value(pv[q], t) * pv[q];
            const T tc = (k > t) ? h.tau * (pv[t] + h.scale * d) : T(0);
            s_tc[t][k] = tc;
            if (k == 0) {
              s_scal[t][0] = h.scale; s_scal[t][1] = h.beta; s_scal[t][2] = h.tau;
            }
            // explicit pivot rows below row t, then the Gram rows of the later columns of the round
#pragma unroll
            for (int q = t + 1; q < S; ++q) pv[q] -= tc * (h.scale * round_lane_value(pv[q], t));
            const T g_tt = hidden2;
#pragma unroll
            for (int i = t + 1; i < S; ++i) {
              const T g_it = round_lane_value(g[i], t);
              const T tc_i = round_lane_value(tc, i);
              const T first = tc * h.scale * g_it, second = tc_i * h.scale * g[t];
              const T third = tc_i * tc * h.scale * h.scale * g_tt;
              g[i] = g[i] - first - second + third;
              if (k == i) size_diag += fabsf(first) + fabsf(second) + fabsf(third);
            }
            accepted = t + 1;
          }
        }
      }
      if (k == 0) {
        s_accepted = accepted;
        s_seen = seen;
      }
    }
    __syncthreads();
    const int accepted = s_accepted;
#pragma unroll
    for (int t = 0; t < S; ++t) {
      if (t < accepted) {
        const T scale = s_scal[t][0], tauv = s_scal[t][2];
        const int jt = j + t;
        // one instruction stream for the rows below the pivot (v = scaled entry), the pivot row
        // (v = 1) and the finished rows above it (v = 0)
        const bool below = r > jt, pivot = r == jt;
        const T v = below ? a[t] * scale : (pivot ? T(1) : T(0));
#pragma unroll
        for (int k = t + 1; k < NB; ++k) a[k] -= s_tc[t][k] * v;
        if (live && pivot) tau[jt] = tauv;
        if (live) {
          // Column jt is final.  Both copies get the reflector in clean form (unit diagonal, zeros
          // above it inside the panel's square top block): the entries of R on and above the
          // diagonal of that block are dropped, the factorisation has no reader for them, and the
          // panel's columns in A can then stand in for V in V^T [V | rest of the block].
          const T vclean = below ? v : (pivot ? T(1) : T(0));
          A[r + (int64_t)jt * lda] = vclean;
          vout[(r - vrow0) + (int64_t)(c + t) * ldv] = vclean;
        }
      }
    }
    // shift the row left by the number of finished columns
    for (int q = 0; q < accepted; ++q) shift_left<1>(a);
    c += accepted;
    // No barrier here: the shared arrays of the next round's first phase (s_wave, s_piv_out) were
    // last read before the barrier that follows the mailbox phase, and the arrays read above are
    // rewritten only behind the next such barrier, which every wavefront reaches after this point.
  }
}

// ---- whole panel per exchange -----------------------------------------------------------------
// The same compressed problem as above with a round that covers every remaining column of the
// panel.  The explicit part is the panel's 32 x 32 top block (rows p .. p+31, all owned by the first
// 32 threads of workgroup 0); everything below it is hidden and enters only through its 32 x 32
// Gram matrix, which a wavefront computes on the matrix cores: its 64 rows go through LDS once to
// get from "lane = row" to the operand layout "lane = (row parity, column)", then 32
// v_mfma_f32_32x32x2 instructions (operand a = operand b) accumulate X^T X.  The workgroups exchange
// the upper triangle of that matrix (528 words) and the top block (1024 words) once (all-to-all up
// to 32 workgroups; beyond that in two levels: a workgroup sums its share of the 528 values over
// all workgroups, publishes the totals, and every workgroup fetches the totals), every
// workgroup runs all Householder steps of the panel on [top block ; Gram] with the same guard as
// above (a round ends before a column whose corrected norm has lost three quarters of its terms'
// size, and that column opens a new round with a freshly computed Gram matrix), and then applies
// the accepted reflectors to its rows.
constexpr int kQrGramWords = kQrNb * (kQrNb + 1) / 2;

// Entry `idx` of the packed upper triangle -> (i, k), i <= k.  Rows i and 31 - i together have 33
// entries, so the triangle is 16 row pairs of 33.
__device__ __forceinline__ void gram_unpack_index(int idx, int& i, int& k) {
  const int pair = idx / (kQrNb + 1), off = idx - pair * (kQrNb + 1);
  if (off < kQrNb - pair) {
    i = pair;
    k = pair + off;
  } else {
    i = kQrNb - 1 - pair;
    k = i + (off - (kQrNb - pair));
  }
}

// Mailbox layout of the Gram values: nine chunks of 64 values, inside a chunk one 64-word row per
// workgroup, so that the words one thread sums (one value, all workgroups) lie 512 bytes apart.
constexpr int kQrGramChunks = (kQrGramWords + 63) / 64;
constexpr int kQrGramMailWords = kQrGramChunks * 64;  // per workgroup
__device__ __forceinline__ size_t gram_mail_offset(int idx, int wg) {
  return ((size_t)(idx >> 6) * kQrPersistentMaxWg + wg) * 64 + (idx & 63);
}

// Workgroup barrier that orders LDS traffic only: __syncthreads() also waits for every global load
// and store of the wavefront, which would expose the latency of loads issued ahead on purpose.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Value of `v` in lane LANE of the caller's half of the wavefront (lanes 0..31 or 32..63), in every
// lane of that half.  Only issues the instruction: the result may be used after lds_wait_all() and,
// so that the compiler keeps the use there, keep_behind_wait() on it.
template <int LANE>
__device__ __forceinline__ float half_broadcast_issue(float v) {
  float r;
  asm volatile("ds_swizzle_b32 %0, %1 offset:%2" : "=v"(r) : "v"(v), "n"(LANE << 5));  // and 0, or LANE, xor 0
  return r;
}
__device__ __forceinline__ void lds_wait_all() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void keep_behind_wait(float& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void keep_behind_wait(int& v) { asm volatile("" : "+v"(v)); }

template <int T0, int T1, class F>
__device__ __forceinline__ void static_for_by4(F&& f) {
  if constexpr (T0 < T1) {
    f(std::integral_constant<int, T0>{});
    static_for_by4<T0 + 4, T1>(f);
  }
}

template <int T0, int T1, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (T0 < T1) {
    f(std::integral_constant<int, T0>{});
    static_for<T0 + 1, T1>(f);
  }
}

// In-block update of a 32-column panel in one launch: C (rows x nc, ld ldc) <- C - V X with
// X = T^T (V^T C) obtained as in reflector_w2_solve_kernel from the split-K slices of V^T [V | C].
// A workgroup owns 256 rows and kPanelApplyCols columns.  Every workgroup of a column group sums
// the slices and solves for X itself (the same numbers in the same order everywhere: 12 KB per
// slice, a forward substitution of 32 steps with one lane per column), which costs less than a
// launch of its own; the product then runs on the matrix cores with the roles of rows and columns
// swapped, D[column][row] += (-X)^T[column][k] V^T[k][row], so that the lanes of a wavefront walk
// down a column of C and of V (coalesced) and X comes out of LDS.
constexpr int kPanelApplyCols = 64;
constexpr int kSliceBatch = 16;  // slices whose loads are in flight together when the slices of V^T [V | C] are summed

// (bx, by) = the workgroup's row block and column group; `col_first` = the first column of C that is
// updated at all (earlier ones belong to someone else), a multiple of 32.
__device__ __forceinline__ void panel_apply_tile(const float* __restrict__ part, int splits, int64_t slab, int nc,
                                                 const float* __restrict__ tau, const float* __restrict__ V,
                                                 int64_t ldv, float* __restrict__ C, int64_t ldc, int rows, int bx,
                                                 int by, int col_first) {
  using T = float;
  constexpr int M = kQrNb, NC = kPanelApplyCols;
  __shared__ __align__(16) T s_g[M][M];   // s_g[i][l] = (V^T V)[i][l], read for i < l
  __shared__ T s_w[NC][M + 1];            // s_w[c][i] = (V^T C)[i][c] of this column group
  __shared__ T s_xn[M][NC];               // s_xn[k][c] = -X[k][c]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col0 = col_first + by * NC;
  // Rows 64 wave .. 64 wave + 63 of the workgroup: two row tiles by two column tiles of 32 x 32.
  // The tile of C and the rows of V are requested first; they arrive while X is being made.
  const int64_t row_base = (int64_t)bx * 256 + wave * 64;
  const int jr = lane & 31, half = lane >> 5;
  const T tau_lane = tau[jr];  // (requested with the first loads, not where the substitution needs it)
  Mfma<T>::Acc acc[2][2];
  T vb[2][M / 2];
  // (loads are unconditional: a row past the end reads the last row and is not stored; a column group
  // that reaches past the last column takes the slower, tested loads)
  const bool full_cols = col0 + NC <= nc;
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
    const int64_t r = min(row_base + rt * 32 + jr, (int64_t)rows - 1);
    const T* vrow = V + r + (int64_t)half * ldv;
    const T* crow = C + r + (int64_t)(col0 + 4 * half) * ldc;
    if (full_cols) {
#pragma unroll
      for (int ct = 0; ct < 2; ++ct)
#pragma unroll
        for (int v = 0; v < Mfma<T>::NACC; ++v)
          acc[rt][ct][v] = crow[(int64_t)(ct * 32 + 8 * (v >> 2) + (v & 3)) * ldc];  // column col0 + ct * 32 + acc_row(v, lane)
    } else {
#pragma unroll
      for (int ct = 0; ct < 2; ++ct)
#pragma unroll
        for (int v = 0; v < Mfma<T>::NACC; ++v) {
          const int c = col0 + ct * 32 + Mfma<T>::acc_row(v, lane);
          acc[rt][ct][v] = (c < nc) ? C[r + (int64_t)c * ldc] : T(0);
        }
    }
#pragma unroll
    for (int ks = 0; ks < M / 2; ++ks) vb[rt][ks] = vrow[(int64_t)(2 * ks) * ldv];
  }
  {
    // Fixed-order sums over the slices, 16 bytes per load: thread tid takes entries 4 tid .. 4 tid + 3
    // of G (four rows of one column) and two such quadruples of this column group's part of W, which
    // is one contiguous run of 64 x 32 words in a slice.
    const int eg = 4 * tid;
    int offset[3];
    bool inside[3];
    offset[0] = eg;
    inside[0] = true;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int e = eg + 1024 * q, c = col0 + (e >> 5);
      inside[1 + q] = c < nc;
      offset[1 + q] = inside[1 + q] ? (M + col0) * M + e : 0;
    }
    float4 sum[3];
#pragma unroll
    for (int q = 0; q < 3; ++q) sum[q] = make_float4(0.f, 0.f, 0.f, 0.f);
    auto add4 = [](float4& acc4, const float4& x) {
      acc4.x += x.x;
      acc4.y += x.y;
      acc4.z += x.z;
      acc4.w += x.w;
    };
    int z = 0;
    for (; z + 8 <= splits; z += 8) {  // eight slices' loads in flight
      float4 v[8][3];
#pragma unroll
      for (int u = 0; u < 8; ++u)
#pragma unroll
        for (int q = 0; q < 3; ++q) v[u][q] = *reinterpret_cast<const float4*>(part + (int64_t)(z + u) * slab + offset[q]);
#pragma unroll
      for (int u = 0; u < 8; ++u)
#pragma unroll
        for (int q = 0; q < 3; ++q) add4(sum[q], v[u][q]);
    }
    for (; z < splits; ++z) {
      float4 v[3];
#pragma unroll
      for (int q = 0; q < 3; ++q) v[q] = *reinterpret_cast<const float4*>(part + (int64_t)z * slab + offset[q]);
#pragma unroll
      for (int q = 0; q < 3; ++q) add4(sum[q], v[q]);
    }
    {
      const int row = eg & 31, col = eg >> 5;
      s_g[row][col] = sum[0].x;
      s_g[row + 1][col] = sum[0].y;
      s_g[row + 2][col] = sum[0].z;
      s_g[row + 3][col] = sum[0].w;
    }
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int e = eg + 1024 * q, row = e & 31, col = e >> 5;
      const float4 t = inside[1 + q] ? sum[1 + q] : make_float4(0.f, 0.f, 0.f, 0.f);
      s_w[col][row] = t.x;
      s_w[col][row + 1] = t.y;
      s_w[col][row + 2] = t.z;
      s_w[col][row + 3] = t.w;
    }
  }
  __syncthreads();
  if (wave == 0) {
    // x_i = tau_i (w_i - sum_{l < i} G[l][i] x_l), one lane per column.  G comes out of registers
    // (lane l holds column l of G; an entry is read across lanes into a scalar): with the entries
    // in LDS every pair of multiply-adds waited for its own LDS read.
    T w[M], gcol[M];
#pragma unroll
    for (int i = 0; i < M; ++i) {
      w[i] = s_w[lane][i];
      gcol[i] = s_g[i][lane & 31];
    }
    static_for<0, M>([&](auto step) {
      constexpr int i = decltype(step)::value;
      const T xi = lane_value<i>(tau_lane) * w[i];
      s_xn[i][lane] = -xi;
      static_for<i + 1, M>([&](auto col) {
        constexpr int l = decltype(col)::value;
        w[l] -= lane_value<l>(gcol[i]) * xi;
      });
    });
  }
  __syncthreads();
#pragma unroll
  for (int ks = 0; ks < M / 2; ++ks) {
    const int k = 2 * ks + half;
    T a[2];
#pragma unroll
    for (int ct = 0; ct < 2; ++ct) a[ct] = s_xn[k][ct * 32 + jr];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int ct = 0; ct < 2; ++ct) acc[rt][ct] = Mfma<T>::mma(a[ct], vb[rt][ks], acc[rt][ct]);
  }
#pragma unroll
  for (int rt = 0; rt < 2; ++rt)
#pragma unroll
    for (int ct = 0; ct < 2; ++ct) {
      const int64_t r = row_base + rt * 32 + jr;
#pragma unroll
      for (int v = 0; v < Mfma<T>::NACC; ++v) {
        const int c = col0 + ct * 32 + Mfma<T>::acc_row(v, lane);
        if (r < rows && c < nc) C[r + (int64_t)c * ldc] = acc[rt][ct][v];
      }
    }
}

__global__ __launch_bounds__(256) void panel_apply_kernel(const float* __restrict__ part, int splits, int64_t slab,
                                                          int nc, const float* __restrict__ tau,
                                                          const float* __restrict__ V, int64_t ldv,
                                                          float* __restrict__ C, int64_t ldc, int rows) {
  panel_apply_tile(part, splits, slab, nc, tau, V, ldv, C, ldc, rows, blockIdx.x, blockIdx.y, 0);
}

// The panel before this one in the same outer block, when its in-block update rides along in this
// launch (`slices` null: it does not).  The first `apply_wgs` workgroups of the grid then update
// the columns behind this panel with the earlier panel's reflectors (panel_apply_tile; they wait for
// nobody), and the panel's own workgroups first bring their 32 columns up to date themselves, in
// registers, from the same slices.  Before a panel workgroup reads the columns behind the panel (for
// its own slice product) it waits until `done_counter` has reached `done_target`, i.e. until every
// updating workgroup of this launch has finished; the counter only ever grows, so it needs no reset.
struct PanelCarry {
  const float* slices;   // the earlier panel's slices of V^T [V | C]
  int splits;            // number of slices
  int64_t slab;          // words per slice
  int nc;                // columns of C behind the earlier panel (the first 32 are this panel)
  const float* tau;      // the earlier panel's 32 tau
  const float* v;        // its reflectors, element (row p of this panel, column 0); ld ldv
  int apply_wgs, apply_row_blocks;
  unsigned* done_counter;
  unsigned done_target;
};

__global__ __launch_bounds__(256) void qr_panel_gram_kernel(float* __restrict__ A, int64_t lda, int n, int p, int pe,
                                                            unsigned long long* part, unsigned long long* piv,
                                                            float* __restrict__ tau, unsigned seq_base, int* error,
                                                            int nwg, unsigned spin_limit, float* __restrict__ vout,
                                                            int64_t ldv, int vrow0, float* __restrict__ slices, int nc,
                                                            int64_t slab, PanelCarry carry) {
  using T = float;
  // Rows of the outer block above this panel: zero in the reflector buffer and in A (the entries of
  // R there have no reader), so that the block's columns of A hold V in clean form as well.  Nobody
  // in this launch reads them; the first updating workgroup does it when it has finished (it has time
  // to spare), the first panel workgroup only when the launch has no updating workgroups.
  auto zero_above_panel = [&]() {
    const int above = p - vrow0;
    for (int col = 0; col < pe - p; ++col)
      for (int row = threadIdx.x; row < above; row += 256) {
        vout[row + (int64_t)col * ldv] = T(0);
        A[(vrow0 + row) + (int64_t)(p + col) * lda] = T(0);
      }
  };
  if (carry.slices != nullptr && (int)blockIdx.x < carry.apply_wgs) {
    // ---- the earlier panel's update of the columns behind this panel ----
    const int bx = (int)blockIdx.x % carry.apply_row_blocks, by = (int)blockIdx.x / carry.apply_row_blocks;
    panel_apply_tile(carry.slices, carry.splits, carry.slab, carry.nc, carry.tau, carry.v, ldv,
                     A + p + (int64_t)p * lda, lda, n - p, bx, by, kQrNb);
    // make the columns visible to the whole device, then count this workgroup as done
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) __hip_atomic_fetch_add(carry.done_counter, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    if (blockIdx.x == 0) zero_above_panel();
    return;
  }
  constexpr int NB = kQrNb, GW = kQrGramWords, XS = NB + 1;
  static_assert(GW == 512 + 16, "the exchange below splits the Gram values as 2 x 256 + 16");
  __shared__ T s_x[4][64 * XS];  // a wavefront's rows on their way to the MFMA layout, then its Gram matrix
  __shared__ T s_sum[4][NB * NB];  // the wavefronts' parts of a 32 x 32 block of V^T [V | C]
  __shared__ T s_tot[NB * NB];   // s_tot[i * NB + k] = G[i][k], both triangles
  __shared__ T s_piv[NB * XS];   // s_piv[q * XS + k] = entry k of row p + q
  __shared__ T s_tc[NB][NB];
  __shared__ T s_scal[NB][2];    // scale, tau of the panel's reflectors
  __shared__ T s_l3[16][16];     // partial sums of the last 16 Gram values, [value][workgroup residue]
  __shared__ T s_seen;           // largest squared column norm of this panel so far
  __shared__ int s_done;
  __shared__ int s_fail;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wg = (int)blockIdx.x - (carry.slices != nullptr ? carry.apply_wgs : 0);
  const int r = p + wg * 256 + tid;
  const int nbw = pe - p;
  const bool live = r < n;
  const bool hidden = live && wg * 256 + tid >= NB;
  if (tid == 0) {
    s_fail = 0;
    s_seen = T(0);
  }
  if (wg == 0 && !(carry.slices != nullptr && carry.apply_wgs > 0)) zero_above_panel();

  T a[NB];  // a[k] = A[r, p + k]
  // (unconditional loads on clamped addresses, zeroed afterwards by clear_unused: tested loads compile
  // to a branch each.  The two are separate because the zeroing is the first use of the loaded values:
  // placed right behind the loads it makes the wavefront wait for them there.)
  auto load_own_row = [&]() {
    const T* arow = A + (live ? r : n - 1) + (int64_t)p * lda;
#pragma unroll
    for (int k = 0; k < NB; ++k) a[k] = arow[(int64_t)min(k, nbw - 1) * lda];
  };
  auto clear_unused = [&]() {
#pragma unroll
    for (int k = 0; k < NB; ++k) a[k] = (live && k < nbw) ? a[k] : T(0);
  };

  if (carry.slices == nullptr) {
    load_own_row();
    clear_unused();
  } else {
    // ---- this panel's columns brought up to date with the earlier panel's reflectors ----
    // a[c] -= sum_t V[r][t] X[t][c], X = T^T (V^T C) for the first 32 columns of C, from the slices
    // as in panel_apply_tile: fixed-order sums (16-byte loads), then the forward substitution with
    // one lane per column.  Every workgroup computes the same X.
    __shared__ __align__(16) T s_cg[NB][NB];   // s_cg[i][l] = (V^T V)[i][l]
    __shared__ T s_cw[NB][NB + 1];             // s_cw[c][i] = (V^T C)[i][c]
    __shared__ __align__(16) T s_cx[NB][NB];   // s_cx[t][c] = -X[t][c]
    // The product runs on the matrix cores as in panel_apply_tile (operand b = V with lane = row of a
    // 32-row tile, requested now and used after X is known).
    const int jr = lane & 31, half = lane >> 5;
    // (requested with the first loads: read where the substitution needs it, it would be one more
    // trip to memory behind the slices)
    const T tau_lane = carry.tau[jr];
    T vb[2][NB / 2];
    // Order of the requests: the slices first, the reflectors and this thread's own row behind them.
    // A wavefront can have 63 loads outstanding and they return in order; with the 64 loads of V and
    // of the row in front, the slices' loads were only issued once those had come back, a second
    // trip to memory before the sums could start.  V and the row are not needed before the
    // substitution is over.
    {
      const int eg = 4 * tid;  // entries 4 tid .. 4 tid + 3 of G, and of the first 32 columns of W
      const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
      float4 sg = zero4, sw = zero4;
      auto add4 = [](float4& acc4, const float4& x) {
        acc4.x += x.x;
        acc4.y += x.y;
        acc4.z += x.z;
        acc4.w += x.w;
      };
      // All batches are full: a slice index past the end reads the last slice again and adds zero
      // (a shorter last batch, or a loop over the remaining slices, would wait for memory once more
      // per slice).
      for (int z = 0; z < carry.splits; z += kSliceBatch) {
        float4 vg[kSliceBatch], vw[kSliceBatch];
#pragma unroll
        for (int u = 0; u < kSliceBatch; ++u) {
          const float* base = carry.slices + (int64_t)min(z + u, carry.splits - 1) * carry.slab;
          vg[u] = *reinterpret_cast<const float4*>(base + eg);
          vw[u] = *reinterpret_cast<const float4*>(base + NB * NB + eg);
        }
#pragma unroll
        for (int u = 0; u < kSliceBatch; ++u) {
          const bool past = z + u >= carry.splits;
          add4(sg, past ? zero4 : vg[u]);
          add4(sw, past ? zero4 : vw[u]);
        }
      }
      const int row = eg & (NB - 1), col = eg >> 5;
      s_cg[row][col] = sg.x;
      s_cg[row + 1][col] = sg.y;
      s_cg[row + 2][col] = sg.z;
      s_cg[row + 3][col] = sg.w;
      s_cw[col][row] = sw.x;
      s_cw[col][row + 1] = sw.y;
      s_cw[col][row + 2] = sw.z;
      s_cw[col][row + 3] = sw.w;
    }
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      const int rl = min(wg * 256 + wave * 64 + rt * 32 + jr, n - 1 - p);  // row of the tile, relative to row p
      const T* vp = carry.v + rl + (int64_t)half * ldv;
#pragma unroll
      for (int ks = 0; ks < NB / 2; ++ks) vb[rt][ks] = vp[(int64_t)(2 * ks) * ldv];
    }
    load_own_row();
    lds_barrier();  // (not __syncthreads(): that would wait for the loads just issued)
    if (wave == 0) {
      T w[NB];
#pragma unroll
      for (int i = 0; i < NB; ++i) w[i] = s_cw[lane & (NB - 1)][i];
      static_for<0, NB>([&](auto step) {
        constexpr int i = decltype(step)::value;
        const T xi = lane_value<i>(tau_lane) * w[i];
        s_cx[i][lane & (NB - 1)] = -xi;  // (both halves of the wavefront hold the same 32 columns)
        static_for<i + 1, NB>([&](auto col) {
          constexpr int l = decltype(col)::value;
          w[l] -= s_cg[i][l] * xi;  // (one address for all lanes: a broadcast read, four entries per instruction)
        });
        // (the updates of a step stay in that step)
        static_for<i + 1, NB>([&](auto col) { keep_behind_wait(w[decltype(col)::value]); });
      });
    }
    lds_barrier();
    {
      // A thread holds its row in a[0..31]; the accumulator layout of a 32 x 32 tile gives lane l
      // columns 8 j + i and lane l + 32 columns 8 j + 4 + i (j, i < 4) of row l.  Swapping the upper
      // half of the registers of one column set with the lower half of the other's turns the two
      // layouts into each other: before the products, and back after them.
      Mfma<T>::Acc acc[2];
#pragma unroll
      for (int v = 0; v < Mfma<T>::NACC; ++v) {
        const int c0 = 8 * (v >> 2) + (v & 3);
        unsigned lo = __float_as_uint(a[c0]), hi = __float_as_uint(a[c0 + 4]);
        lane_swap<true>(lo, hi);
        acc[0][v] = __uint_as_float(lo);  // rows 0..31 of the wavefront
        acc[1][v] = __uint_as_float(hi);  // rows 32..63
      }
#pragma unroll
      for (int ks = 0; ks < NB / 2; ++ks) {
        const T xk = s_cx[2 * ks + half][jr];
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) acc[rt] = Mfma<T>::mma(xk, vb[rt][ks], acc[rt]);
      }
#pragma unroll
      for (int v = 0; v < Mfma<T>::NACC; ++v) {
        const int c0 = 8 * (v >> 2) + (v & 3);
        unsigned lo = __float_as_uint(acc[0][v]), hi = __float_as_uint(acc[1][v]);
        lane_swap<true>(lo, hi);
        a[c0] = __uint_as_float(lo);
        a[c0 + 4] = __uint_as_float(hi);
      }
    }
    clear_unused();
  }

  int c = 0;  // finished columns
  for (unsigned round = 0; c < nbw; ++round) {
    const unsigned seq = seq_base + round + 1u;
    unsigned long long* part_c = part + (size_t)(round & 1) * kQrPersistentMaxWg * kQrGramMailWords;
    unsigned long long* piv_c = piv + (round & 1) * NB * NB;
    // What the steps below compare and address with is made opaque once per round.  As loop invariants
    // the 32 masks `t < nbw`, the 64 masks `r > p + t`, `r == p + t` and the 64 column addresses were
    // all computed in front of the loop (which usually runs once) and kept in spill lanes and
    // accumulator registers until their step: 2000 instructions per launch.
    int nbw_r = nbw, p_r = p, rel_r = wg * 256 + tid;  // (rel_r: this thread's row, counted from row p)
    int64_t lda_r = lda, ldv_r = ldv;
    // (the pointers themselves stay as they are: behind an asm statement the compiler no longer knows
    // that they point to global memory, and its generic stores also count as LDS traffic)
    asm volatile("" : "+s"(nbw_r), "+s"(p_r), "+s"(lda_r), "+s"(ldv_r));
    asm volatile("" : "+v"(rel_r));
    // the top block first: it is on its way while the Gram matrix is being computed (column by column,
    // 256 contiguous bytes per store instruction: with a row per lane, 32 scattered words each, the
    // 32 stores took 4 us to issue)
    if (wg == 0 && tid < NB) {
#pragma unroll
      for (int k = 0; k < NB; ++k)
        __hip_atomic_store(piv_c + k * NB + tid, mailbox_pack(live ? a[k] : T(0), seq), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
    // Gram matrix of this wavefront's hidden rows (finished columns ride along; nobody reads them)
    {
      T* xs = s_x[wave];
#pragma unroll
      for (int k = 0; k < NB; ++k) xs[lane * XS + k] = hidden ? a[k] : T(0);
      lds_barrier();  // (the barriers of this loop order LDS traffic only; __syncthreads() would also wait for the mailbox stores)
      Mfma<T>::Acc acc = {}, acc_odd = {};  // two chains, so that an instruction need not wait for the one before it
#pragma unroll
      for (int s = 0; s < 32; s += 2) {
        const T x0 = xs[(2 * s + (lane >> 5)) * XS + (lane & 31)];
        const T x1 = xs[(2 * s + 2 + (lane >> 5)) * XS + (lane & 31)];
        acc = Mfma<T>::mma(x0, x0, acc);
        acc_odd = Mfma<T>::mma(x1, x1, acc_odd);
      }
      acc += acc_odd;
      // (a wavefront's LDS accesses complete in order: its reads above are done before these writes)
#pragma unroll
      for (int v = 0; v < Mfma<T>::NACC; ++v) xs[Mfma<T>::acc_row(v, lane) * NB + (lane & 31)] = acc[v];
    }
    lds_barrier();
    for (int idx = tid; idx < GW; idx += 256) {
      int i, k;
      gram_unpack_index(idx, i, k);
      const int e = i * NB + k;
      const T sum = (s_x[0][e] + s_x[1][e]) + (s_x[2][e] + s_x[3][e]);
      __hip_atomic_store(part_c + gram_mail_offset(idx, wg), mailbox_pack(sum, seq), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    }
    {
      // Fixed-order sums over the workgroups.  Up to 32 workgroups thread tid takes the values tid and
      // tid + 256 over all workgroups; the 16 values from 512 on are split sixteen ways over the
      // workgroups (thread tid: value 512 + tid % 16, workgroups tid / 16, tid / 16 + 16, ...).
      bool ok = true;
      T sum[2] = {T(0), T(0)}, sum3 = T(0);
      const unsigned long long* base3 = part_c + gram_mail_offset(512 + (tid & 15), tid >> 4);
      const int count3 = (nwg - (tid >> 4) + 15) >> 4;  // workgroups tid / 16, tid / 16 + 16, ... below nwg
      float top_value[4] = {0.f, 0.f, 0.f, 0.f};
      if (nwg <= 32) {
        // one trip to memory for the lot (three in the general form below: the two values one after
        // the other, then the top block; with more than 32 workgroups, where a thread has over a
        // hundred loads to make either way, the single trip was no faster)
        const unsigned long long* base0 = part_c + gram_mail_offset(tid, 0);
        const unsigned long long* base1 = part_c + gram_mail_offset(tid + 256, 0);
        if (nwg <= 16)
          ok = mailbox_wait_all<16, 1>(base0, base1, nwg, base3, count3, piv_c + tid, seq, error, spin_limit, sum[0], sum[1],
                                       sum3, top_value);
        else
          ok = mailbox_wait_all<32, 2>(base0, base1, nwg, base3, count3, piv_c + tid, seq, error, spin_limit, sum[0], sum[1],
                                       sum3, top_value);
      } else {
        // More workgroups: two levels.  All-to-all, every workgroup would read the 528 values of every
        // other one (8 MB per exchange at 43 workgroups, 10 us on the fabric between the XCDs).
        // Level 1: this workgroup sums its share of the values, `per` consecutive ones, over all
        // workgroups (one thread per value, workgroups in ascending order) and publishes the totals;
        // level 2: every thread fetches the totals it needs, and its words of the top block.
        const int per = (GW + nwg - 1) / nwg;  // (at most 16)
        unsigned long long* total_c =
            part + (size_t)2 * kQrPersistentMaxWg * kQrGramMailWords + (size_t)(round & 1) * kQrGramMailWords;
        const int mine = wg * per + tid;
        if (tid < per && mine < GW) {
          T total = T(0), unused = T(0);
          for (int w0 = 0; w0 < nwg && ok; w0 += 32)  // (a batch may reach past the last workgroup: spare rows)
            ok = mailbox_wait_sum<32, 64, 0, 1>(part_c + gram_mail_offset(mine, w0), nwg - w0, part_c, 0, seq, error,
                                                spin_limit, total, unused);
          if (ok) __hip_atomic_store(total_c + mine, mailbox_pack(total, seq), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (ok) {
          const unsigned long long* slot[7];
          const bool used[7] = {true, true, true, true, true, true, true};
          float v[7];
          slot[0] = total_c + tid;
          slot[1] = total_c + 256 + tid;
          slot[2] = total_c + 512 + (tid & 15);
#pragma unroll
          for (int u = 0; u < 4; ++u) slot[3 + u] = piv_c + tid + 256 * u;
          ok = mailbox_wait<7>(slot, used, seq, error, spin_limit, v);
          sum[0] = v[0];
          sum[1] = v[1];
          sum3 = (tid < 16) ? v[2] : T(0);  // (s_l3 holds sixteen partial sums per value: here one of them is the total)
#pragma unroll
          for (int u = 0; u < 4; ++u) top_value[u] = v[3 + u];
        }
      }
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        int i, k;
        gram_unpack_index(tid + 256 * half, i, k);
        s_tot[i * NB + k] = sum[half];
        s_tot[k * NB + i] = sum[half];
      }
      s_l3[tid & 15][tid >> 4] = sum3;
#pragma unroll
      for (int u = 0; u < 4; ++u)
        s_piv[(tid & (NB - 1)) * XS + (tid >> 5) + 8 * u] = top_value[u];  // word k * NB + q of the mail
      if (!ok) {
        __hip_atomic_store(error, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_fail = 1;
      }
    }
    lds_barrier();
    if (s_fail) return;
    if (tid < 16) {
      T total = T(0);
#pragma unroll
      for (int u = 0; u < 16; ++u) total += s_l3[tid][u];
      int i, k;
      gram_unpack_index(512 + tid, i, k);
      s_tot[i * NB + k] = total;
      s_tot[k * NB + i] = total;
    }
    lds_barrier();
    if (wave == 0) {
      // Lanes 0..31 hold the top block E, lanes 32..63 the Gram matrix G: lane k of either half owns
      // column k of its matrix (x[q] = entry q).  A step needs entry q of column t of E in every lane
      // of the lower half and entry q of column t of G (= G[t][q], its symmetric twin) in every lane
      // of the upper half: one broadcast inside each half of the wavefront serves both, and one
      // instruction stream updates both matrices,
      //   E[q][k] -= tc_k (E[q][t] s)
      //   G[q][k] -= tc_k (G[q][t] s) + tc_q u_k,   u_k = s G[t][k] - tc_k s^2 G[t][t]
      // (the correction <a'_q,a'_k> = <a_q,a_k> - tc_k s<a_t,a_q> - tc_q s<a_t,a_k> + tc_q tc_k s^2<a_t,a_t>).
      const int k = lane & (NB - 1);
      const bool upper = lane >= NB;
      T x[NB];
#pragma unroll
      for (int q = 0; q < NB; ++q) x[q] = upper ? s_tot[q * NB + k] : s_piv[q * XS + k];
      T size_diag = fabsf(s_tot[k * NB + k]);  // size of the terms G[k][k] is made of (same in both halves)
      T seen = s_seen;
      int done = c;
      bool open = true;
      // Straight-line code per step: once a step has been refused (`open` false) the later steps
      // still run, on numbers nobody will use - the rows' owners apply only the steps before `done`,
      // and the next round starts from their rows.
      static_for<0, NB>([&](auto step) {
        constexpr int t = decltype(step)::value;
        if (t >= c && t < nbw_r) {
          // (the lane's column number and half are made opaque per step: otherwise the compiler keeps
          // the 32 masks `k > t` and the half masks live across the whole panel in scalar registers it
          // does not have, and reloads each from a spill slot with two cross-lane reads)
          int kk = k, half = upper ? 1 : 0;
          keep_behind_wait(kk);
          keep_behind_wait(half);
          const bool upper_t = half != 0;
          // b[q] = entry q of column t, broadcast over the half.  All broadcasts of a step are issued
          // together and waited for once (the compiler, left to place them, waits for each one where
          // it is used).
          T b[NB];
          static_for<t + 1, NB>([&](auto row) {
            constexpr int q = decltype(row)::value;
            b[q] = half_broadcast_issue<t>(x[q]);
          });
          lds_wait_all();
          static_for<t + 1, NB>([&](auto row) {
            constexpr int q = decltype(row)::value;
            keep_behind_wait(b[q]);
          });
          // lower half: e_k = <column t, column k> of E over the rows below pivot t
          T e = T(0);
          static_for<t + 1, NB>([&](auto row) {
            constexpr int q = decltype(row)::value;
            e += b[q] * x[q];
          });
          // Both halves need E[t][k], G[t][k] and e_k: a swap of the halves of two copies of a
          // register leaves the lower half's value in every lane of one and the upper half's in
          // every lane of the other.
          unsigned xt_lower = __float_as_uint(x[t]), xt_upper = xt_lower;
          lane_swap<true>(xt_lower, xt_upper);
          unsigned e_lower = __float_as_uint(e), e_upper = e_lower;
          lane_swap<true>(e_lower, e_upper);
          const T pvt = __uint_as_float(xt_lower);  // E[t][k]
          const T gt = __uint_as_float(xt_upper);   // G[t][k]
          const T ek = __uint_as_float(e_lower);
          const T alpha = lane_value<t>(pvt);
          const T hidden2 = lane_value<t>(gt);
          const T x2_explicit = lane_value<t>(ek);
          const T size_t_ = lane_value<t>(size_diag);
          // (the last column of the matrix has nothing below its pivot: exactly zero, so tau = 0 as in LAPACK)
          const T x2 = (p_r + t < n - 1) ? x2_explicit + fmaxf(hidden2, T(0)) : T(0);
          const bool finite = hidden2 - hidden2 == T(0);
          open = open && (t == c || (finite && alpha * alpha + x2 >= kQrRoundGuard * size_t_));
          const Reflector h = make_reflector_fast(alpha, x2, kQrNegligible * seen);
          seen = open ? fmaxf(seen, alpha * alpha + x2) : seen;  // (what outlives the round must not see a refused step)
          const T d = gt + ek;  // <column t, column k> below pivot t
          const T tc = (kk > t) ? h.tau * (pvt + h.scale * d) : T(0);
          if (!upper_t) s_tc[t][k] = tc;
          s_scal[t][0] = h.scale;  // (every lane writes the same two numbers)
          s_scal[t][1] = h.tau;
          const T w = h.scale * gt;
          const T s2gtt = h.scale * h.scale * hidden2;
          const T u = upper_t ? w - tc * s2gtt : T(0);
          static_for<t + 1, NB>([&](auto row) {
            constexpr int q = decltype(row)::value;
            // lower half: rounded exactly as the rows' owners do it further down, so that both hold
            // the same numbers (u = 0 there; lane t itself has tc = 0).  This matters: with the scale
            // folded into tc once per step (one multiplication less per entry, results a rounding
            // apart) the factorisation of a matrix with pairs of nearly equal columns lost its
            // backward stability.
            x[q] = (x[q] - tc * (b[q] * h.scale)) - lane_value<q>(tc) * u;
          });
          size_diag += T(2) * fabsf(tc * w) + fabsf(tc * tc * s2gtt);
          done = open ? t + 1 : done;
        }
      });
      if (lane == 0) {
        s_done = done;
        s_seen = seen;
      }
    }
    lds_barrier();
    const int done = s_done;
    // The rows' owners apply the steps [c, done).  One instruction stream for the rows below the pivot
    // (v = scaled entry), the pivot row (v = 1) and the finished rows above it (v = 0); the finished
    // column's register then holds this row of V (nothing reads it before the end).  The usual case,
    // a whole panel in one round, runs without a test per step, so that the coefficients of the next
    // step are on their way from LDS while this one is applied; nothing is stored before all steps
    // are done.
    auto apply_step = [&](auto step) {
      constexpr int t = decltype(step)::value;
      const T scale = s_scal[t][0];
      const bool below = rel_r > t, pivot = rel_r == t;
      const T v = below ? a[t] * scale : (pivot ? T(1) : T(0));
#pragma unroll
      for (int k = t + 1; k < NB; ++k) a[k] -= s_tc[t][k] * v;
      a[t] = v;
    };
    const bool whole = c == 0 && done == NB;
    if (whole) {
      static_for<0, NB>(apply_step);
    } else {
      static_for<0, NB>([&](auto step) {
        constexpr int t = decltype(step)::value;
        if (t >= c && t < done) apply_step(step);
      });
    }
    if (wg == 0 && tid < NB && tid >= c && tid < done && live) tau[p_r + tid] = s_scal[tid][1];
    if (live) {
      // clean form in both copies, as in the kernel above; the addresses walk from column to column
      T* acol = A + r + (int64_t)p_r * lda_r;
      T* vcol = vout + (r - vrow0);
      if (whole) {
#pragma unroll
        for (int t = 0; t < NB; ++t) {
          *acol = a[t];
          *vcol = a[t];
          acol += lda_r;
          vcol += ldv_r;
        }
      } else {
        static_for<0, NB>([&](auto step) {
          constexpr int t = decltype(step)::value;
          if (t >= c && t < done) {
            *acol = a[t];
            *vcol = a[t];
          }
          acol += lda_r;
          vcol += ldv_r;
        });
      }
    }
    c = done;
  }
  if (slices == nullptr) return;
  if (carry.slices != nullptr && carry.apply_wgs > 0) {
    // the columns behind the panel are being updated by the first workgroups of this launch
    if (tid == 0) {
      unsigned polls = 0;
      bool ok = true;
      while (__hip_atomic_load(carry.done_counter, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) - carry.done_target >
             0x7fffffffu) {  // (counter still behind the target, in wrap-around arithmetic)
        if (++polls > spin_limit) {
          ok = false;
          break;
        }
        __builtin_amdgcn_s_sleep(2);
      }
      if (!ok) {
        __hip_atomic_store(error, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_fail = 1;
      }
    }
    __syncthreads();
    if (s_fail) return;
    __threadfence();
  }
  // ---- this workgroup's slice of V^T [V | C] ------------------------------------------------------
  // C = the nc columns behind the panel (the rest of the outer block), V = the panel's reflectors,
  // both over this workgroup's 256 rows.  The in-block update needs the sums of these slices over
  // the workgroups; computing them here saves a launch that would read V and C again.  A wavefront
  // multiplies its own 64 rows: V goes through LDS once into the "b" operand layout (32 registers),
  // each 32-column block of C is loaded row per lane (256 contiguous bytes per instruction), passed
  // through the same LDS area into the "a" layout and multiplied with 32 v_mfma_f32_32x32x2; the four
  // wavefronts' results are added through LDS in a fixed order.  Block 0 is V^T V.
  // Slice layout: element (i, j) of the 32 x (32 + nc) matrix at slices[wg * slab + i + 32 * j].
  {
    T* xs = s_x[wave];
    const int half = lane >> 5, l31 = lane & 31;
    const int blocks = 1 + (nc + NB - 1) / NB;
    // Loads are unconditional on clamped addresses (a row past the end reads the last row, a column
    // past the end the last column): such rows have V = 0 and such columns are not stored.  The
    // column's base address is the same for all lanes, the row a 32-bit index.
    const int rr = live ? r : n - 1;
    // Two blocks of C are on their way at any time (block jb covers columns 32 (jb - 1) ...): the
    // matrix was just written by other workgroups, so a block's loads come from memory, which takes
    // longer than the products of one block.
    T cur[2][NB];
    auto load_block = [&](T (&dst)[NB], int jb) {
      const int c0 = (jb - 1) * NB;
      const T* base = A + (int64_t)(pe + c0) * lda;
      if (c0 + NB <= nc) {
#pragma unroll
        for (int k = 0; k < NB; ++k) dst[k] = base[(int64_t)k * lda + rr];
      } else {
#pragma unroll
        for (int k = 0; k < NB; ++k) dst[k] = base[(int64_t)min(k, nc - 1 - c0) * lda + rr];
      }
    };
    if (blocks > 1) load_block(cur[0], 1);  // on their way while V is staged and V^T V computed
    if (blocks > 2) load_block(cur[1], 2);
#pragma unroll
    for (int k = 0; k < NB; ++k) xs[lane * XS + k] = a[k];
    T vb[NB];
#pragma unroll
    for (int s = 0; s < NB; ++s) vb[s] = xs[(2 * s + half) * XS + l31];
    auto emit = [&](int jb, const Mfma<T>::Acc& acc) {
#pragma unroll
      for (int v = 0; v < Mfma<T>::NACC; ++v) s_sum[wave][Mfma<T>::acc_row(v, lane) * NB + l31] = acc[v];
      lds_barrier();
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int e = tid + 256 * q;  // i = e % 32, j = 32 jb + e / 32
        if (jb * NB + (e >> 5) < NB + nc)
          slices[(int64_t)wg * slab + jb * (NB * NB) + e] = (s_sum[0][e] + s_sum[1][e]) + (s_sum[2][e] + s_sum[3][e]);
      }
      lds_barrier();
    };
    {
      Mfma<T>::Acc acc = {}, acc_odd = {};
#pragma unroll
      for (int s = 0; s < NB; s += 2) {
        acc = Mfma<T>::mma(vb[s], vb[s], acc);
        acc_odd = Mfma<T>::mma(vb[s + 1], vb[s + 1], acc_odd);
      }
      acc += acc_odd;
      emit(0, acc);
    }
    auto multiply_block = [&](T (&src)[NB], int jb) {
      // (a wavefront's LDS accesses complete in order: the reads of the block before are done)
#pragma unroll
      for (int k = 0; k < NB; ++k) xs[lane * XS + k] = src[k];
      if (jb + 2 < blocks) load_block(src, jb + 2);  // into the registers just emptied
      T x[NB];
#pragma unroll
      for (int s = 0; s < NB; ++s) x[s] = xs[(2 * s + half) * XS + l31];
      Mfma<T>::Acc acc = {}, acc_odd = {};
#pragma unroll
      for (int s = 0; s < NB; s += 2) {
        acc = Mfma<T>::mma(x[s], vb[s], acc);
        acc_odd = Mfma<T>::mma(x[s + 1], vb[s + 1], acc_odd);
      }
      acc += acc_odd;
      emit(jb, acc);
    };
    for (int jb = 1; jb < blocks; jb += 2) {
      multiply_block(cur[0], jb);
      if (jb + 1 < blocks) multiply_block(cur[1], jb + 1);
    }
  }
}

// Vc (nrows x nbw, ld ldv) <- the unit-lower-trapezoidal reflector block stored in A, column c with
// its unit entry in row c + shift of the block: zeros above, one there, A[row0 + i, col0 + c] below.
// shift = 0: QR reflectors (unit diagonal at (row0 + c, col0 + c)); shift = 1: the reflectors of a
// tridiagonalisation, which start one row below the diagonal (row 0 of the block is then all zero).
template <typename T>
__global__ void extract_v_kernel(const T* __restrict__ A, int64_t lda, int nrows, int row0, int col0, int nbw,
                                 T* __restrict__ Vc, int64_t ldv, int shift) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;  // row within the block
  if (i >= nrows) return;
  for (int c = blockIdx.y; c < nbw; c += gridDim.y) {
    T v;
    if (i < c + shift) v = T(0);
    else if (i == c + shift) v = T(1);
    else v = A[(row0 + i) + (int64_t)(col0 + c) * lda];
    Vc[i + (int64_t)c * ldv] = v;
  }
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
// G may arrive as `splits` unreduced split-K slices (`slab` elements apart), summed while loading:
// the block's 32 (double: 4) groups of 32 threads take slices z = group, group + groups, ... (all
// loads of a thread are in flight together), and the groups' sums are then added in a fixed order through LDS.
template <typename T>
constexpr int larft_groups() {
  return sizeof(T) == 8 ? 4 : 32;  // double (already summed input only): 128 threads, all registers for the recursion
}

template <typename T>
__global__ __launch_bounds__(32 * larft_groups<T>()) void larft32_kernel(const T* __restrict__ G, int ldg, int splits,
                                                                    int64_t slab, const T* __restrict__ tau, int nbw,
                                                                    T* __restrict__ Tm, int ldt) {
  constexpr int STAGE = sizeof(T) == 8 ? 4 : 8;  // groups that exchange through LDS at a time (33 KB)
  constexpr int kLarftGroups = larft_groups<T>();
  __shared__ T s_g[STAGE][32][33];
  const int b = blockIdx.x;
  const int w = min(32, nbw - 32 * b);
  G += (int64_t)32 * b * (ldg + 1);
  Tm += (int64_t)32 * b * (ldt + 1);
  tau += 32 * b;
  const int k = threadIdx.x & 31, zg = threadIdx.x >> 5;
  T t[32], g[32];
#pragma unroll
  for (int c = 0; c < 32; ++c) g[c] = T(0);
  if (k < w) {
    for (int z = zg; z < splits; z += kLarftGroups) {
      const T* slice = G + (int64_t)z * slab + k;
#pragma unroll
      for (int c = 0; c < 32; ++c) g[c] += (c < w) ? slice[c * ldg] : T(0);
    }
  }
  if (splits > 1) {
    // groups STAGE .. 31 hand their sums to groups 0 .. STAGE-1, STAGE groups at a time
    for (int base = STAGE; base < kLarftGroups && base < splits; base += STAGE) {
      if (zg >= base && zg < base + STAGE) {
#pragma unroll
        for (int c = 0; c < 32; ++c) s_g[zg - base][k][c] = g[c];
      }
      __syncthreads();
      if (zg < STAGE && zg + base < splits) {
#pragma unroll
        for (int c = 0; c < 32; ++c) g[c] += s_g[zg][k][c];
      }
      __syncthreads();
    }
    if (zg > 0 && zg < STAGE) {
#pragma unroll
      for (int c = 0; c < 32; ++c) s_g[zg][k][c] = g[c];
    }
    __syncthreads();
    if (zg == 0) {
      for (int q = 1; q < STAGE && q < splits; ++q) {
#pragma unroll
        for (int c = 0; c < 32; ++c) g[c] += s_g[q][k][c];
      }
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

// Fills the diagonal of Q with NaN if the error flag is set, and raises the host-visible report
// word (pinned host memory, may be null) so that the host can learn of the failure without
// reading Q.
template <typename T>
__global__ void poison_on_error_kernel(T* __restrict__ Q, int64_t ldq, int n, const int* __restrict__ error,
                                       int* __restrict__ report) {
  if (*error == 0) return;
  for (int i = threadIdx.x; i < n; i += blockDim.x) Q[i + (int64_t)i * ldq] = T(NAN);
  if (report && threadIdx.x == 0) *report = 1;
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
// the rest of Tm must be zero).  The blocks above the diagonal follow by doubling: two neighbouring
// spans of S reflectors with factors T11 and T22 have the joint factor [T11 T12; 0 T22] with
// T12 = -T11 (G12 T22); all pairs of one span length are independent and share a launch, so a
// 256-wide factor takes three levels (S = 32, 64, 128) of two products each.
template <typename T>
static inline int assemble_t_factor_ld(hipStream_t s, const T* gram, int ldg, T* mx, int ldmx, int nbw, const T* tau,
                                       T* Tm, int ldt, int first_block) {
  using Small = typename SmallTile<T>::type;
  const int blocks = (int)ceil_div64(nbw, 32);
  if (first_block < blocks) {
    hipLaunchKernelGGL((larft32_kernel<T>), dim3(blocks - first_block), dim3(32 * larft_groups<T>()), 0, s,
                       gram + (int64_t)32 * first_block * (ldg + 1), ldg, 1, (int64_t)0, tau + 32 * first_block,
                       nbw - 32 * first_block, Tm + (int64_t)32 * first_block * (ldt + 1), ldt);
    SOAPMI_LAUNCH_CHECK();
  }
  for (int S = 32; S < nbw; S *= 2) {
    // from one pair's blocks to the next pair's; block (0, S) and (S, S) of a pair relative to its block (0, 0)
    const int64_t pair_g = (int64_t)2 * S * (ldg + 1), pair_t = (int64_t)2 * S * (ldt + 1);
    const int64_t pair_m = (int64_t)2 * S * (ldmx + 1);
    const int64_t g12 = (int64_t)S * ldg, t12 = (int64_t)S * ldt, t22 = (int64_t)S * (ldt + 1), m12 = (int64_t)S * ldmx;
    const int full = nbw / (2 * S);              // pairs whose right span is complete
    const int right = nbw - (2 * S * full + S);  // width of the last, shorter right span (<= 0: none)
    int rc = gemm_strided_batch<T, Small>(s, S, S, S, T(1), gram + g12, ldg, pair_g, Tm + t22, ldt, pair_t, T(0),
                                          mx + m12, ldmx, pair_m, full);
    if (rc) return rc;
    rc = gemm_strided_batch<T, Small>(s, S, S, S, T(-1), Tm, ldt, pair_t, mx + m12, ldmx, pair_m, T(0), Tm + t12, ldt,
                                      pair_t, full);
    if (rc) return rc;
    if (right > 0) {
      rc = gemm<T, Small>(s, 0, 0, S, right, right, T(1), gram + full * pair_g + g12, ldg, Tm + full * pair_t + t22, ldt,
                          T(0), mx + full * pair_m + m12, ldmx);
      if (rc) return rc;
      rc = gemm<T, Small>(s, 0, 0, S, right, S, T(-1), Tm + full * pair_t, ldt, mx + full * pair_m + m12, ldmx, T(0),
                          Tm + full * pair_t + t12, ldt);
      if (rc) return rc;
    }
  }
  return kOk;
}

template <typename T>
static inline int assemble_t_factor(hipStream_t s, const BlockReflectorWs<T>& ws, int nbw, const T* tau, T* Tm,
                                    int first_block) {
  return assemble_t_factor_ld<T>(s, ws.gram, kBrMax, ws.mx, kBrMax, nbw, tau, Tm, kBrMax, first_block);
}

// Number of K slices for a tall-skinny product with `tiles` output tiles, K = rows, an M x N
// output.  Slices have at least 128 rows and the partial results must fit the split-K buffer
// (kBrSplits * kBrMax * ldv elements).  With a handful of tiles: as many slices as it takes to
// occupy the chip (about 512 workgroups).  With more tiles the workgroups of a launch are spread
// over the 256 CUs and a CU works through its share one after the other, so the time goes as
// ceil(tiles * slices / 256) / slices: the slice count that minimises it is taken (fewest slices
// among near-equal ones), which avoids launches whose last CU round is nearly empty.
static inline int split_count(int64_t tiles, int rows, int M, int N, int64_t ldv) {
  if (rows < 512) return 1;
  const int64_t capacity = (int64_t)kBrSplits * kBrMax * ldv / std::max<int64_t>(1, (int64_t)M * N);
  const int64_t most = std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(capacity, 64), rows / 128));
  if (tiles <= 8) return (int)std::min<int64_t>(ceil_div64(512, tiles), most);
  int best = 1;
  double best_cost = (double)ceil_div64(tiles, 256);
  for (int64_t slices = 2; slices <= std::min<int64_t>(most, 16); ++slices) {
    const double cost = (double)ceil_div64(tiles * slices, 256) / (double)slices;
    if (cost < 0.97 * best_cost) {
      best = (int)slices;
      best_cost = cost;
    }
  }
  return best;
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

// W2 (M x N, ld ldw2) = T^T W for a panel of M <= 32 reflectors without forming T: the inverse of the
// compact-WY factor is known in closed form, T^-1 = strict upper triangle of V^T V + diag(1 / tau),
// so T^T W is the solution X of a lower triangular system, x_i = tau_i (w_i - sum_{l<i} G[l][i] x_l).
// `part` holds the split-K slices of V^T [V | C] (M rows, ld M): columns 0..M-1 are G = V^T V,
// column M + c is column c of W = V^T C.  A reflector with tau = 0 (none) gets x_i = 0, as its
// zero row and column of T would give.  256 threads = 8 groups of 32 lanes, one column of W per
// group: everyone sums G's slices into LDS (fixed order), each group sums and substitutes its column.
constexpr int kW2SolveCols = 8;

template <typename T>
__global__ __launch_bounds__(256) void reflector_w2_solve_kernel(const T* __restrict__ part, int splits, int64_t slab,
                                                                 int M, int N, const T* __restrict__ tau,
                                                                 T* __restrict__ W2, int ldw2) {
  __shared__ T s_g[32][33];
  const int tid = threadIdx.x, l = tid & 31, group = tid >> 5;
  const int c = blockIdx.x * kW2SolveCols + group;
  {
    // entry e = tid + 256 q of the M x M block G (column-major, ld M); out-of-range entries read
    // element 0 and are zeroed afterwards, so that the loads carry no branch
    int offset[4];
    bool inside[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int e = tid + 256 * q, row = e & 31, col = e >> 5;
      inside[q] = row < M && col < M;
      offset[q] = inside[q] ? row + col * M : 0;
    }
    T g[4] = {T(0), T(0), T(0), T(0)};
    int z = 0;
    for (; z + 8 <= splits; z += 8) {
      T v[8][4];
#pragma unroll
      for (int u = 0; u < 8; ++u)
#pragma unroll
        for (int q = 0; q < 4; ++q) v[u][q] = part[(int64_t)(z + u) * slab + offset[q]];
#pragma unroll
      for (int u = 0; u < 8; ++u)
#pragma unroll
        for (int q = 0; q < 4; ++q) g[q] += v[u][q];
    }
    for (; z < splits; ++z)
#pragma unroll
      for (int q = 0; q < 4; ++q) g[q] += part[(int64_t)z * slab + offset[q]];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int e = tid + 256 * q;
      s_g[e & 31][e >> 5] = inside[q] ? g[q] : T(0);
    }
  }
  const bool mine = l < M && c < N;
  T w = T(0);
  {
    const T* column = part + (mine ? l + (int64_t)(M + c) * M : 0);
    int z = 0;
    for (; z + 8 <= splits; z += 8) {
      T v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = column[(int64_t)(z + u) * slab];
#pragma unroll
      for (int u = 0; u < 8; ++u) w += v[u];
    }
    for (; z < splits; ++z) w += column[(int64_t)z * slab];
    if (!mine) w = T(0);
  }
  __syncthreads();
  const T tau_l = (l < M) ? tau[l] : T(0);
  T x = T(0);
  for (int i = 0; i < M; ++i) {
    const T xi = __shfl(tau_l * w, i, 32);  // final for lane i: every l < i has been subtracted
    if (l == i) x = xi;
    if (l > i) w -= s_g[i][l] * xi;
  }
  if (mine) W2[l + (int64_t)c * ldw2] = x;
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

// The same for the trailing columns of a factorisation whose panel kernels left V in clean form in
// the block's own columns of A as well: those columns and the trailing ones are neighbours in A, so
// one product gives V^T [V | C], i.e. the Gram matrix the T factor is built from and W.
// `block` = element (first row, first column) of the outer block in A; T (ld kBrMax) is assembled here.
template <typename T>
static inline int factor_and_apply_block_reflector(hipStream_t s, const BlockReflectorWs<T>& ws, T* Tm, int rows,
                                                   int nbw, int nc, int64_t ldv, T* block, int64_t lda, const T* tau,
                                                   int first_block) {
  using Wide = typename DefaultTile<T>::type;
  const int64_t tiles = ceil_div64(nbw + nc, Wide::BN) * ceil_div64(nbw, Wide::BM);
  const int splits = split_count(tiles, rows, nbw, nbw + nc, ldv);
  int rc = gemm<T>(s, 1, 0, nbw, nbw + nc, rows, T(1), ws.v, ldv, block, lda, T(0), ws.w, kBrMax, splits, ws.splitk);
  if (rc) return rc;
  BlockReflectorWs<T> gram_in_w = ws;
  gram_in_w.gram = ws.w;
  rc = assemble_t_factor<T>(s, gram_in_w, nbw, tau, Tm, first_block);
  if (rc || nc <= 0) return rc;
  rc = gemm<T>(s, 1, 0, nbw, nc, nbw, T(1), Tm, kBrMax, ws.w + (int64_t)nbw * kBrMax, kBrMax, T(0), ws.w2, kBrMax);
  if (rc) return rc;
  return gemm<T>(s, 0, 0, rows, nc, nbw, T(-1), ws.v, ldv, ws.w2, kBrMax, T(1), block + (int64_t)nbw * lda, lda);
}

template <typename T>
static inline void launch_extract_v(hipStream_t s, const T* A, int64_t lda, int rows, int row0, int col0, int nbw,
                                    T* V, int64_t ldv, int shift = 0) {
  hipLaunchKernelGGL((extract_v_kernel<T>), dim3((unsigned)ceil_div64(rows, 256), (unsigned)std::min(nbw, 32)),
                     dim3(256), 0, s, A, lda, rows, row0, col0, nbw, V, ldv, shift);
}

// State of the panel chain that runs through a whole factorisation.
struct QrChainState {
  unsigned seq_base = 0;       // sequence number of the next panel's first column (mailbox tags)
  unsigned carried_total = 0;  // updating workgroups issued so far (what ws.sync[2] counts up to)
};

template <typename T>
struct QrWorkspace;

// The 32-column panels of the outer block [P, PE) of A (n x n): each panel is factored and applied
// to the rest of the outer block.  Tm (ld kBrMax) receives diagonal 32-blocks of the outer factor
// only on the launch-per-column path (*inner_done counts them).
template <typename T>
static inline int qr_outer_block_panels(hipStream_t s, T* A, int64_t lda, int n, int P, int PE, T* Tm,
                                        const QrWorkspace<T>& ws, int persistent_max_wg, unsigned spin_limit,
                                        int columns_per_round, bool carry_updates, QrChainState* chain,
                                        int* inner_done, bool* v_written, bool* clean_in_a);

// ---- QR driver -------------------------------------------------------------------------------
// Mailbox words per workgroup and for the pivot rows: the larger of what the two persistent panel
// kernels use (four columns per round: 4 x 32 and 4 x 32; whole panel: 9 x 64 and 32 x 32).
constexpr int kQrMailWords = kQrGramMailWords > kQrRoundMax * kQrNb ? kQrGramMailWords : kQrRoundMax * kQrNb;
constexpr int kQrMailPivotWords = kQrNb * kQrNb;
// behind the mailboxes: the totals of the whole-panel kernel's two-level exchange (2 x 576 words), and room
// for its batched loads, which read up to 31 rows past the last workgroup, used or not
constexpr int kQrMailSpareWords = 48 * 64;
constexpr int kQrWholePanel = kQrNb;  // columns_per_round value that selects qr_panel_gram_kernel
constexpr int kQrSuper = 1024;        // widest super-block (third blocking level of the factorisation)

template <typename T>
struct QrWorkspace {
  BlockReflectorWs<T> br;
  T* t_all;   // outer blocks x kBrMax x kBrMax
  T* tau;     // n
  T* part;    // 2 x nwg x NB   partials of the launch-per-column fallback
  T* piv;     // 2 x NB
  unsigned long long* mail_part;  // 2 x kQrPersistentMaxWg x kQrMailWords   mailboxes of the persistent panel kernels
  unsigned long long* mail_piv;   // 2 x kQrMailPivotWords
  unsigned* sync;  // [1] error flag of the persistent panel kernel, [2] count of finished updating workgroups
  // third blocking level: super-blocks of up to kQrSuper columns (leading dimension sb_ld of all five)
  int sb_ld;
  T* t_super;  // super-blocks x sb_ld x sb_ld   compact-WY factors of the super-blocks
  T* gram_s;   // sb_ld x sb_ld   row band k: V_k^T [V_0 .. V_k | C] of the super-block's k-th outer block
  T* mx_s;     // sb_ld x sb_ld
  T* w_s;      // sb_ld x n
  T* w2_s;     // sb_ld x n
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
  q.mail_part = ws.template take<unsigned long long>((size_t)2 * kQrPersistentMaxWg * kQrMailWords + kQrMailSpareWords);
  q.mail_piv = ws.template take<unsigned long long>(2 * kQrMailPivotWords);
  q.sync = ws.template take<unsigned>(64);
  // (padded: with a power of two as leading dimension the columns of T, W and W2 that a product
  // reads together lie 4 KB apart and collide in the caches: measured 17 TFLOP/s for T^T W)
  q.sb_ld = (int)std::min<int64_t>(kQrSuper, blocks * kBrMax) + 32;
  q.t_super = ws.template take<T>((size_t)ceil_div64(n, kQrSuper) * q.sb_ld * q.sb_ld);
  q.gram_s = ws.template take<T>((size_t)q.sb_ld * q.sb_ld);
  q.mx_s = ws.template take<T>((size_t)q.sb_ld * q.sb_ld);
  q.w_s = ws.template take<T>((size_t)q.sb_ld * n);
  q.w2_s = ws.template take<T>((size_t)q.sb_ld * n);
  if (out) *out = q;
}

template <typename T>
static inline size_t qr_workspace_bytes(int64_t n) {
  WorkspaceSizer sizer;
  qr_workspace_layout<T>(sizer, n, nullptr);
  return sizer.total();
}

template <typename T>
static inline int qr_outer_block_panels(hipStream_t s, T* A, int64_t lda, int n, int P, int PE, T* Tm,
                                        const QrWorkspace<T>& ws, int persistent_max_wg, unsigned spin_limit,
                                        int columns_per_round, bool carry_updates, QrChainState* chain,
                                        int* inner_done, bool* v_written, bool* clean_in_a) {
  const int NB = kQrNb, OB = kBrMax;
  const int64_t ldv = n;
  int rc;
  int pending_p = -1, pending_nwg = 0, pending_buffer = 0;  // a panel whose in-block update has not been issued
  for (int p = P; p < PE; p += NB) {
    const int pe = std::min(PE, p + NB), nbw = pe - p;
    const int rows = n - p;
    const int nwg = (int)ceil_div64(rows, 256);
    T* part[2] = {ws.part, ws.part + (size_t)nwg * NB};
    T* piv[2] = {ws.piv, ws.piv + NB};
    // this panel's reflectors inside the outer block's n x 128 buffer (origin: row P, column P)
    BlockReflectorWs<T> inner = ws.br;
    inner.v = ws.br.v + (p - P) + (int64_t)(p - P) * ldv;
    bool slices_by_panel = false;
    if (nwg <= persistent_max_wg && columns_per_round == kQrWholePanel) {
      // (a full panel with columns of the outer block behind it also leaves its slices of V^T [V | C];
      // two slice buffers alternate, since a launch may read the earlier panel's while writing its own)
      slices_by_panel = pe < PE && nbw == NB;
      T* slice_buffer[2] = {ws.br.splitk, ws.br.splitk + (size_t)kBrSplits * kBrMax * ldv / 2};
      PanelCarry carry{};
      if (pending_p >= 0 && nbw == NB) {
        // the earlier panel's in-block update rides along in this launch
        const int groups = (int)ceil_div64(PE - pe, kPanelApplyCols);
        carry.slices = slice_buffer[pending_buffer];
        carry.splits = pending_nwg;
        carry.slab = (int64_t)NB * (PE - pending_p);
        carry.nc = PE - p;
        carry.tau = ws.tau + pending_p;
        carry.v = ws.br.v + (p - P) + (int64_t)(pending_p - P) * ldv;
        carry.apply_row_blocks = nwg;
        carry.apply_wgs = nwg * groups;
        carry.done_counter = ws.sync + 2;
        chain->carried_total += (unsigned)carry.apply_wgs;
        carry.done_target = chain->carried_total;
        pending_p = -1;
      } else if (pending_p >= 0) {
        // (a last, narrower panel: the earlier panel's update as a launch of its own)
        hipLaunchKernelGGL(panel_apply_kernel,
                           dim3((unsigned)ceil_div64(n - pending_p, 256), (unsigned)ceil_div64(PE - p, kPanelApplyCols)),
                           dim3(256), 0, s, slice_buffer[pending_buffer], pending_nwg, (int64_t)NB * (PE - pending_p),
                           PE - p, ws.tau + pending_p, ws.br.v + (pending_p - P) + (int64_t)(pending_p - P) * ldv, ldv,
                           A + pending_p + (int64_t)p * lda, lda, n - pending_p);
        SOAPMI_LAUNCH_CHECK();
        pending_p = -1;
      }
      const int out_buffer = pending_buffer ^ 1;
      hipLaunchKernelGGL(qr_panel_gram_kernel, dim3(nwg + carry.apply_wgs), dim3(256), 0, s, A, lda, n, p, pe,
                         ws.mail_part, ws.mail_piv, ws.tau, chain->seq_base, reinterpret_cast<int*>(ws.sync + 1), nwg, spin_limit,
                         ws.br.v + (int64_t)(p - P) * ldv, ldv, P, slices_by_panel ? slice_buffer[out_buffer] : nullptr,
                         PE - pe, (int64_t)NB * (PE - p), carry);
      chain->seq_base += (unsigned)nbw;
      if (slices_by_panel) {
        pending_buffer = out_buffer;
        if (carry_updates) {
          pending_p = p;
          pending_nwg = nwg;
        } else {
          hipLaunchKernelGGL(panel_apply_kernel,
                             dim3((unsigned)nwg, (unsigned)ceil_div64(PE - pe, kPanelApplyCols)), dim3(256), 0, s,
                             slice_buffer[out_buffer], nwg, (int64_t)NB * (PE - p), PE - pe, ws.tau + p, inner.v, ldv,
                             A + p + (int64_t)pe * lda, lda, rows);
        }
      }
    } else if (nwg <= persistent_max_wg) {
      *clean_in_a = false;
      hipLaunchKernelGGL(qr_panel_persistent_kernel, dim3(nwg), dim3(256), 0, s, A, lda, n, p, pe, ws.mail_part,
                         ws.mail_piv, ws.tau, chain->seq_base, reinterpret_cast<int*>(ws.sync + 1), nwg, spin_limit,
                         ws.br.v + (int64_t)(p - P) * ldv, ldv, P, columns_per_round);
      chain->seq_base += (unsigned)nbw;
    } else {
      for (int j = p - 1; j < pe; ++j) {
        const int in = (j - p + 1) & 1, out = in ^ 1;
        hipLaunchKernelGGL((qr_panel_step_kernel<T>), dim3(nwg), dim3(256), 0, s, A, lda, n, p, pe, j, part[in],
                           piv[in], part[out], piv[out], ws.tau, nwg);
      }
      *v_written = false;
      *clean_in_a = false;
    }
    SOAPMI_LAUNCH_CHECK();
    if (slices_by_panel) {
      // (the in-block update is on its way or rides along with the next panel)
    } else if (pe < PE && *v_written) {
      // The panel's reflectors act on the rest of the outer block only.  One product gives the
      // slices of V^T [V | C] (the panel's own columns of A hold V in clean form); the middle
      // factor T^T is applied as a triangular solve with V^T V, so no T is needed here: the
      // diagonal blocks of the outer factor are all built after the block's last panel.
      using Skinny = typename SkinnyTile<T>::type;
      const int ncols = PE - p, nc = PE - pe;
      int slices = 1;
      rc = gemm_to_partials<T, Skinny>(s, 1, 0, nbw, ncols, rows, inner.v, ldv, A + p + (int64_t)p * lda, lda,
                                       split_count(ceil_div64(ncols, Skinny::BN), rows, nbw, ncols, ldv),
                                       ws.br.splitk, &slices);
      if (rc) return rc;
      if (nbw == NB) {
        hipLaunchKernelGGL(panel_apply_kernel, dim3((unsigned)ceil_div64(rows, 256), (unsigned)ceil_div64(nc, kPanelApplyCols)),
                           dim3(256), 0, s, ws.br.splitk, slices, (int64_t)nbw * ncols, nc, ws.tau + p, inner.v, ldv,
                           A + p + (int64_t)pe * lda, lda, rows);
        SOAPMI_LAUNCH_CHECK();
      } else {
        hipLaunchKernelGGL((reflector_w2_solve_kernel<T>), dim3((unsigned)ceil_div64(nc, kW2SolveCols)), dim3(256), 0, s,
                           ws.br.splitk, slices, (int64_t)nbw * ncols, nbw, nc, ws.tau + p, ws.br.w2, kBrMax);
        SOAPMI_LAUNCH_CHECK();
        rc = gemm<T>(s, 0, 0, rows, nc, nbw, T(-1), inner.v, ldv, ws.br.w2, kBrMax, T(1), A + p + (int64_t)pe * lda, lda);
        if (rc) return rc;
      }
    } else if (pe < PE) {
      T* Tin = Tm + (int64_t)(p - P) * (OB + 1);  // diagonal block of the outer factor
      launch_extract_v<T>(s, A, lda, rows, p, p, nbw, inner.v, ldv);
      int slices = 1;  // V^T V stays in split-K slices; the factor kernel sums them while loading
      rc = gemm_to_partials<T, typename SkinnyTile<T>::type>(s, 1, 0, nbw, nbw, rows, inner.v, ldv, inner.v, ldv,
                                                             split_count(1, rows, nbw, nbw, ldv), inner.splitk,
                                                             &slices);
      if (rc) return rc;
      hipLaunchKernelGGL((larft32_kernel<T>), dim3(1), dim3(32 * larft_groups<T>()), 0, s, inner.splitk, nbw, slices,
                         (int64_t)nbw * nbw, ws.tau + p, nbw, Tin, OB);
      SOAPMI_LAUNCH_CHECK();
      rc = apply_block_reflector<T>(s, inner, Tin, true, rows, nbw, PE - pe, ldv, A + p + (int64_t)pe * lda, lda);
      if (rc) return rc;
      ++*inner_done;
    }
  }
  return kOk;
}

// geqrf in place on A (n x n), then the explicit Q into Qout (n x n).  A is destroyed.
// Two levels of blocking: 32-column panels (register-resident column steps) are applied only
// inside their kBrMax-column outer block; the trailing matrix and Q see kBrMax-wide block
// reflectors, whose products have K = kBrMax and run on the full-size MFMA tile.
template <typename T>
static inline int qr_factor_and_form_q_two_level(hipStream_t s, T* A, int64_t lda, T* Qout, int64_t ldq, int n,
                                                 const QrWorkspace<T>& ws, int persistent_max_wg, unsigned spin_limit,
                                                 int columns_per_round, int* report, bool carry_updates) {
  const int NB = kQrNb, OB = kBrMax;
  const int blocks = (int)ceil_div64(n, OB);
  const int64_t ldv = n;
  int rc;
  static_assert(std::is_same<T, float>::value, "the persistent panel kernel packs float values into its mailboxes");
  QrChainState chain;
  std::vector<char> block_clean((size_t)blocks, 0);  // outer blocks whose columns of A hold V in clean form
  hipLaunchKernelGGL((fill_zero_kernel<unsigned>), dim3(1), dim3(64), 0, s, ws.sync, 64);
  {
    // sequence number 0 = "nothing yet"; mail_piv follows mail_part in the workspace, one clear covers both
    const int words = (int)(reinterpret_cast<unsigned*>(ws.mail_piv + 2 * kQrMailPivotWords) -
                            reinterpret_cast<unsigned*>(ws.mail_part));
    hipLaunchKernelGGL((fill_zero_kernel<unsigned>), dim3((words + 255) / 256), dim3(256), 0, s,
                       reinterpret_cast<unsigned*>(ws.mail_part), words);
  }
  // (the T factors of all outer blocks start from zero: one fill instead of one per block)
  hipLaunchKernelGGL((fill_zero_kernel<T>), dim3(blocks * (OB * OB / 256)), dim3(256), 0, s, ws.t_all, blocks * OB * OB);
  // ---- factorisation ----
  for (int bi = 0; bi < blocks; ++bi) {
    const int P = bi * OB, PE = std::min(n, P + OB), obw = PE - P;
    T* Tm = ws.t_all + (size_t)bi * OB * OB;
    int inner_done = 0;
    bool v_written = true;   // the panel kernels leave the block's reflectors in ws.br.v
    bool clean_in_a = true;  // every panel left V in clean form in A too (the whole-panel kernel does)
    rc = qr_outer_block_panels<T>(s, A, lda, n, P, PE, Tm, ws, persistent_max_wg, spin_limit, columns_per_round,
                                  carry_updates, &chain, &inner_done, &v_written, &clean_in_a);
    if (rc) return rc;
    const int rows = n - P;
    if (!v_written) launch_extract_v<T>(s, A, lda, rows, P, P, obw, ws.br.v, ldv);
    block_clean[bi] = clean_in_a ? 1 : 0;
    if (clean_in_a && obw > kQrNb) {
      // T and the trailing columns, C <- H^T C = C - V T^T V^T C, from one product V^T [V | C]
      rc = factor_and_apply_block_reflector<T>(s, ws.br, Tm, rows, obw, n - PE, ldv, A + P + (int64_t)P * lda, lda,
                                               ws.tau + P, inner_done);
      if (rc) return rc;
    } else {
      rc = gram_of_v<T>(s, ws.br, rows, obw, ldv);
      if (rc) return rc;
      rc = assemble_t_factor<T>(s, ws.br, obw, ws.tau + P, Tm, inner_done);
      if (rc) return rc;
      // trailing columns: C <- H^T C = C - V T^T V^T C
      rc = apply_block_reflector<T>(s, ws.br, Tm, true, rows, obw, n - PE, ldv, A + P + (int64_t)PE * lda, lda);
      if (rc) return rc;
    }
  }
  // ---- explicit Q, outer blocks in reverse ----
  for (int bi = blocks - 1; bi >= 0; --bi) {
    const int P = bi * OB, PE = std::min(n, P + OB), obw = PE - P;
    const int rows = n - P;
    T* Tm = ws.t_all + (size_t)bi * OB * OB;
    // V of the block: its columns of A where the panel kernels left them in clean form, else extracted
    BlockReflectorWs<T> bws = ws.br;
    int64_t ldvb = ldv;
    if (block_clean[bi] && lda == ldv) {  // (the split-K buffer is sized by the reflector buffer's leading dimension)
      bws.v = A + P + (int64_t)P * lda;
      ldvb = lda;
    } else {
      launch_extract_v<T>(s, A, lda, rows, P, P, obw, ws.br.v, ldv);
      SOAPMI_LAUNCH_CHECK();
    }
    // columns to the right already hold Q of the later blocks: C <- (I - V T V^T) C
    rc = apply_block_reflector<T>(s, bws, Tm, false, rows, obw, n - PE, ldvb, Qout + P + (int64_t)PE * ldq, ldq);
    if (rc) return rc;
    // own columns: [I;0] - V (T V1^T)
    rc = gemm<T>(s, 0, 1, obw, obw, obw, T(1), Tm, OB, bws.v, ldvb, T(0), ws.br.mx, OB);
    if (rc) return rc;
    rc = gemm<T>(s, 0, 0, rows, obw, obw, T(-1), bws.v, ldvb, ws.br.mx, OB, T(0), Qout + P + (int64_t)P * ldq, ldq);
    if (rc) return rc;
    hipLaunchKernelGGL((orgqr_panel_fix_kernel<T>), dim3((unsigned)ceil_div64(PE, 256)), dim3(256), 0, s, Qout, ldq, P,
                       obw);
    SOAPMI_LAUNCH_CHECK();
  }
  // A panel kernel that gave up waiting leaves garbage behind: make that impossible to miss.
  hipLaunchKernelGGL((poison_on_error_kernel<T>), dim3(1), dim3(64), 0, s, Qout, ldq, n,
                     reinterpret_cast<const int*>(ws.sync + 1), report);
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

// Zeroes, in the columns of the super-block [S0, S1) of A, the rows of the super-block above each
// outer block's own rows (entries of R that no one reads), so that the super-block's columns hold
// its reflectors in clean form from row S0 on.  Grid: (row chunks of 256, outer blocks 1 ..).
template <typename T>
__global__ __launch_bounds__(256) void zero_above_blocks_kernel(T* __restrict__ A, int64_t lda, int S0, int S1) {
  const int P = S0 + kBrMax * ((int)blockIdx.y + 1), PE = min(S1, P + kBrMax);
  const int r = S0 + (int)blockIdx.x * 256 + (int)threadIdx.x;
  if (r >= P) return;
  for (int c = P; c < PE; ++c) A[r + (int64_t)c * lda] = T(0);
}

// Slice count of a product with a long K whose partial results go to the block-reflector split-K
// buffer (`capacity` elements).
static inline int split_count_capacity(int64_t tiles, int rows, int M, int N, int64_t capacity) {
  // split_count sizes by kBrSplits * kBrMax * ldv: hand it the ldv that gives `capacity`
  return split_count(tiles, rows, M, N, capacity / ((int64_t)kBrSplits * kBrMax));
}

// C (rows x nc, ld ldc) <- (I - V op(T) V^T) C for a reflector block of any width k (V rows x k in
// clean form; T k x k upper triangular, ld ldt); W and W2 (k x nc, ld ldw) are scratch.
template <typename T>
static inline int apply_wide_reflector(hipStream_t s, const T* V, int64_t ldv, const T* Tm, int ldt, bool transT,
                                       int rows, int k, int nc, T* C, int64_t ldc, T* W, T* W2, int ldw, T* splitk,
                                       int64_t splitk_capacity) {
  using Wide = typename DefaultTile<T>::type;
  if (nc <= 0 || rows <= 0 || k <= 0) return kOk;
  const int64_t tiles = ceil_div64(nc, Wide::BN) * ceil_div64(k, Wide::BM);
  const int splits = split_count_capacity(tiles, rows, k, nc, splitk_capacity);
  int rc = gemm<T>(s, 1, 0, k, nc, rows, T(1), V, ldv, C, ldc, T(0), W, ldw, splits, splitk);
  if (rc) return rc;
  rc = gemm<T>(s, transT ? 1 : 0, 0, k, nc, k, T(1), Tm, ldt, W, ldw, T(0), W2, ldw);
  if (rc) return rc;
  return gemm<T>(s, 0, 0, rows, nc, k, T(-1), V, ldv, W2, ldw, T(1), C, ldc);
}

// Three levels of blocking: panels of 32 columns inside outer blocks of kBrMax columns as above, and
// outer blocks inside super-blocks of kQrSuper columns.  An outer block's reflectors are applied only
// to the rest of its super-block; everything beyond sees the super-block as one kQrSuper-wide
// compact-WY reflector, so the bulk of the trailing updates and of the Q formation are products
// with K = kQrSuper, which re-read and re-write the trailing matrix a quarter as often as K = kBrMax
// ones.  The super-block's factor T has the outer blocks' factors on its diagonal and above it
// T12 = -T11 (V1^T V2) T22 by doubling (spans of 256, 512); the cross products V_k^T V_l (l < k) come
// out of the product that an outer block needs anyway, V_k^T A[:, super-block]: its columns left of
// the block are the earlier blocks' reflectors, the block's own columns give V_k^T V_k and the rest
// V_k^T C.  Requires every panel to run on the whole-panel kernel (which leaves V in clean form in A).
template <typename T>
static inline int qr_factor_and_form_q_three_level(hipStream_t s, T* A, int64_t lda, T* Qout, int64_t ldq, int n,
                                                   const QrWorkspace<T>& ws, int persistent_max_wg,
                                                   unsigned spin_limit, int* report, bool carry_updates) {
  using Wide = typename DefaultTile<T>::type;
  const int OB = kBrMax, SB = kQrSuper, LD = ws.sb_ld;
  const int supers = (int)ceil_div64(n, SB);
  const int64_t ldv = n;
  const int64_t splitk_capacity = (int64_t)kBrSplits * kBrMax * n;
  int rc;
  QrChainState chain;
  hipLaunchKernelGGL((fill_zero_kernel<unsigned>), dim3(1), dim3(64), 0, s, ws.sync, 64);
  {
    const int words = (int)(reinterpret_cast<unsigned*>(ws.mail_piv + 2 * kQrMailPivotWords) -
                            reinterpret_cast<unsigned*>(ws.mail_part));
    hipLaunchKernelGGL((fill_zero_kernel<unsigned>), dim3((words + 255) / 256), dim3(256), 0, s,
                       reinterpret_cast<unsigned*>(ws.mail_part), words);
  }
  {
    const int64_t count = (int64_t)supers * LD * LD;
    hipLaunchKernelGGL((fill_zero_kernel<T>), dim3((unsigned)ceil_div64(count, 256)), dim3(256), 0, s, ws.t_super,
                       (int)count);
  }
  SOAPMI_LAUNCH_CHECK();
  // ---- factorisation ----
  for (int si = 0; si < supers; ++si) {
    const int S0 = si * SB, S1 = std::min(n, S0 + SB), sbw = S1 - S0;
    T* Ts = ws.t_super + (size_t)si * LD * LD;
    for (int P = S0; P < S1; P += OB) {
      const int PE = std::min(S1, P + OB), obw = PE - P, rows = n - P;
      T* Tm = Ts + (int64_t)(P - S0) * (LD + 1);  // diagonal block of the super-block's factor
      int inner_done = 0;
      bool v_written = true, clean_in_a = true;
      rc = qr_outer_block_panels<T>(s, A, lda, n, P, PE, (T*)nullptr, ws, persistent_max_wg, spin_limit, kQrWholePanel,
                                    carry_updates, &chain, &inner_done, &v_written, &clean_in_a);
      if (rc) return rc;
      if (!v_written || !clean_in_a || inner_done != 0) {
        set_error("internal error: a QR panel left the whole-panel path");
        return kRuntimeError;
      }
      // row band of the super-block's Gram matrix: V_k^T A[P:, S0:S1]
      T* band = ws.gram_s + (P - S0);
      const int64_t tiles = ceil_div64(sbw, Wide::BN) * ceil_div64(obw, Wide::BM);
      rc = gemm<T>(s, 1, 0, obw, sbw, rows, T(1), ws.br.v, ldv, A + P + (int64_t)S0 * lda, lda, T(0), band, LD,
                   split_count_capacity(tiles, rows, obw, sbw, splitk_capacity), ws.br.splitk);
      if (rc) return rc;
      rc = assemble_t_factor_ld<T>(s, band + (int64_t)(P - S0) * LD, LD, ws.br.mx, kBrMax, obw, ws.tau + P, Tm, LD, 0);
      if (rc) return rc;
      const int nc = S1 - PE;
      if (nc > 0) {  // the rest of the super-block: C <- C - V_k T_k^T (V_k^T C)
        rc = gemm<T>(s, 1, 0, obw, nc, obw, T(1), Tm, LD, band + (int64_t)(PE - S0) * LD, LD, T(0), ws.br.w2, kBrMax);
        if (rc) return rc;
        rc = gemm<T>(s, 0, 0, rows, nc, obw, T(-1), ws.br.v, ldv, ws.br.w2, kBrMax, T(1), A + P + (int64_t)PE * lda, lda);
        if (rc) return rc;
      }
    }
    // blocks of T above the diagonal blocks, by doubling: spans of kBrMax, 2 kBrMax, ...
    for (int S = OB; S < sbw; S *= 2) {
      for (int o = 0; o + S < sbw; o += 2 * S) {
        const int r = std::min(S, sbw - (o + S));  // width of the right span
        const T* g21 = ws.gram_s + (o + S) + (int64_t)o * LD;       // V2^T V1 (r x S)
        const T* t11 = Ts + (int64_t)o * (LD + 1);
        const T* t22 = Ts + (int64_t)(o + S) * (LD + 1);
        T* t12 = Ts + o + (int64_t)(o + S) * LD;
        rc = gemm<T>(s, 1, 0, S, r, r, T(1), g21, LD, t22, LD, T(0), ws.mx_s, LD);
        if (rc) return rc;
        rc = gemm<T>(s, 0, 0, S, r, S, T(-1), t11, LD, ws.mx_s, LD, T(0), t12, LD);
        if (rc) return rc;
      }
    }
    if (sbw > OB) {
      hipLaunchKernelGGL((zero_above_blocks_kernel<T>), dim3((unsigned)ceil_div64(sbw - OB, 256), (unsigned)ceil_div64(sbw - OB, OB)),
                         dim3(256), 0, s, A, lda, S0, S1);
      SOAPMI_LAUNCH_CHECK();
    }
    // everything beyond the super-block: C <- H^T C = C - V T^T V^T C with K = sbw
    rc = apply_wide_reflector<T>(s, A + S0 + (int64_t)S0 * lda, lda, Ts, LD, true, n - S0, sbw, n - S1,
                                 A + S0 + (int64_t)S1 * lda, lda, ws.w_s, ws.w2_s, LD, ws.br.splitk, splitk_capacity);
    if (rc) return rc;
  }
  // ---- explicit Q, super-blocks in reverse ----
  for (int si = supers - 1; si >= 0; --si) {
    const int S0 = si * SB, S1 = std::min(n, S0 + SB), sbw = S1 - S0;
    const T* Ts = ws.t_super + (size_t)si * LD * LD;
    // columns beyond the super-block already hold Q of the later ones: C <- (I - V T V^T) C
    rc = apply_wide_reflector<T>(s, A + S0 + (int64_t)S0 * lda, lda, Ts, LD, false, n - S0, sbw, n - S1,
                                 Qout + S0 + (int64_t)S1 * ldq, ldq, ws.w_s, ws.w2_s, LD, ws.br.splitk, splitk_capacity);
    if (rc) return rc;
    // own columns, all outer blocks at once: [I;0] - V (T V1^T).  (Block by block, each applied to the
    // later columns of the super-block, would be half the arithmetic, in products of a few tiles each
    // that run at a quarter of the rate.)
    const T* V = A + S0 + (int64_t)S0 * lda;
    rc = gemm<T>(s, 0, 1, sbw, sbw, sbw, T(1), Ts, LD, V, lda, T(0), ws.mx_s, LD);
    if (rc) return rc;
    rc = gemm<T>(s, 0, 0, n - S0, sbw, sbw, T(-1), V, lda, ws.mx_s, LD, T(0), Qout + S0 + (int64_t)S0 * ldq, ldq);
    if (rc) return rc;
    hipLaunchKernelGGL((orgqr_panel_fix_kernel<T>), dim3((unsigned)ceil_div64(S1, 256)), dim3(256), 0, s, Qout, ldq, S0,
                       sbw);
    SOAPMI_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL((poison_on_error_kernel<T>), dim3(1), dim3(64), 0, s, Qout, ldq, n,
                     reinterpret_cast<const int*>(ws.sync + 1), report);
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

// geqrf in place on A (n x n), then the explicit Q into Qout (n x n).  A is destroyed.  `super_block`:
// kQrSuper selects the three-level blocking where every panel can run on the whole-panel kernel,
// kBrMax (and every other panel setting) the two-level one, 0 chooses by size.  Measured on MI355X
// (ms, three-level / two-level): n = 1024 1.99 / 2.07, 2048 4.32 / 4.39, 4096 10.30 / 10.40,
// 8192 33.4 / 33.4, 11008 61.2 / 59.7, 14336 107.2 / 106.4.  The K = 1024 products of the explicit Q
// run at 120 TFLOP/s against 101 for K = 256, but the scheme needs about 15 % more arithmetic (T^T W
// with K = 1024, a super-block's own columns of Q as one product), and in the factorisation its
// products arrive in bursts between panel chains, where this GPU gives 100 to 111 TFLOP/s for a
// product that reaches 127 in a steady stream.
constexpr int kQrSuperAutoMax = 4096;  // three levels up to this size when the choice is left to the library
template <typename T>
static inline int qr_factor_and_form_q(hipStream_t s, T* A, int64_t lda, T* Qout, int64_t ldq, int n,
                                       const QrWorkspace<T>& ws, int persistent_max_wg = kQrPersistentMaxWg,
                                       unsigned spin_limit = kQrSpinLimit, int columns_per_round = kQrRoundMax,
                                       int* report = nullptr, bool carry_updates = true, int super_block = 0) {
  if (super_block == 0) super_block = n <= kQrSuperAutoMax ? kQrSuper : kBrMax;
  if (super_block == kQrSuper && columns_per_round == kQrWholePanel && ceil_div64(n, 256) <= persistent_max_wg)
    return qr_factor_and_form_q_three_level<T>(s, A, lda, Qout, ldq, n, ws, persistent_max_wg, spin_limit, report,
                                               carry_updates);
  return qr_factor_and_form_q_two_level<T>(s, A, lda, Qout, ldq, n, ws, persistent_max_wg, spin_limit,
                                           columns_per_round, report, carry_updates);
}

}  // namespace soapmi
