// LDS-tiled MFMA GEMM for gfx950, column-major operands, fp32 (v_mfma_f32_32x32x2_f32) and
// fp64 (v_mfma_f64_16x16x4_f64).  One kernel template serves every matrix product on the SOAP
// path; what differs per call site is the epilogue functor, which receives each accumulator
// element together with its global (m, n) coordinate:
//   EpiStore     C = alpha*acc + beta*C                    (rotations, P*Q, block reflectors)
//   EpiEmaLower  C = lerp(C, acc, w) on the lower triangle (Gram EMA, optional mirror)
//   EpiAdam      Adam moment update + normalised update    (forward rotation, 2nd product)
//   EpiPartial   raw partial sums for split-K              (tall-skinny products)
//
// Data layout.  op(A) is M x K, op(B) is K x N, both stored column-major with a leading
// dimension; "trans" means the stored matrix is the transpose of the operand.  A K-slab of
// each operand is staged in LDS as S[k][x] (x = m or n contiguous), so that the MFMA fragment
// reads of a wavefront are 32 (16) consecutive words.  The MFMA "a" operand is fed from the
// B tile and the "b" operand from the A tile: accumulator lanes then run along m, and every
// epilogue load/store instruction touches 128 consecutive bytes of a column of C.
#pragma once
#include <type_traits>

#include "common.hpp"

#ifndef SOAPMI_TILE_GROUP_ROWS
#define SOAPMI_TILE_GROUP_ROWS 8
#endif

namespace soapmi {

template <typename T>
struct GemmProblem {
  const T* A;
  const T* B;
  int64_t lda, ldb;
  int M, N, K;
  int transA, transB;
  int vecA, vecB;      // 16-byte global loads are legal for this operand
  int tiles_m, tiles_n;
  int num_tiles;
  int lower;           // enumerate only tiles with tile_m >= tile_n (square tile grid)
  int k_chunk;         // K extent handled by one blockIdx.y slice (multiple of BK)
  const int* ksel_b;   // general path, B operand x-contiguous only: row k of op(B) is stored as row ksel_b[k] (null: k)
};

// ---- epilogues ---------------------------------------------------------------------------
template <typename T>
struct EpiStore {
  T* C;
  int64_t ldc;
  T alpha, beta;
  __device__ __forceinline__ void operator()(int m, int n, T v, int) const {
    T* p = C + m + (int64_t)n * ldc;
    T r = alpha * v;
    if (beta != T(0)) r += beta * (*p);
    *p = r;
  }
};

template <typename T>
struct EpiPartial {
  T* part;        // [splits][N][M] compact
  int64_t ld;     // = M
  int64_t slab;   // = M*N
  __device__ __forceinline__ void operator()(int m, int n, T v, int z) const {
    part[(int64_t)z * slab + m + (int64_t)n * ld] = v;
  }
};

template <typename T>
__device__ __forceinline__ T lerp_like_torch(T start, T end, T weight) {
  // Same two-branch form as torch.lerp (used by the reference: preconditioners.py:367,579).
  return (weight < T(0.5)) ? start + weight * (end - start) : end - (end - start) * (T(1) - weight);
}

template <typename T>
struct EpiEmaLower {
  T* C;
  int64_t ldc;
  T weight;    // 1 - beta
  int mirror;  // also write the transposed element so both triangles stay valid
  __device__ __forceinline__ void operator()(int m, int n, T v, int) const {
    if (m < n) return;
    T* p = C + m + (int64_t)n * ldc;
    T r = lerp_like_torch(*p, v, weight);
    *p = r;
    if (mirror && m != n) C[n + (int64_t)m * ldc] = r;
  }
};

struct AdamScalars {
  float beta1, beta2;
  float one_minus_beta1, one_minus_beta2;
  float bias_correction1;       // 1 - beta1^step
  float sqrt_bias_correction2;  // sqrt(1 - beta2^step)
  float eps;                    // already rescaled by the caller (soap.py:367)
};

__device__ __forceinline__ float adam_element(float g, float* mom, float* var, const AdamScalars& s) {
  // Operation order follows optimizer.py:36-44.
  float m = (*mom) * s.beta1 + g * s.one_minus_beta1;
  float v = (*var) * s.beta2 + s.one_minus_beta2 * g * g;
  *mom = m;
  *var = v;
  float denom = sqrtf(v) / s.sqrt_bias_correction2 + s.eps;
  return (1.0f / denom) * m / s.bias_correction1;
}

struct EpiAdam {
  float* mom;
  float* var;
  float* upd;
  int64_t ldm, ldv, ldu;
  AdamScalars s;
  __device__ __forceinline__ void operator()(int m, int n, float g, int) const {
    upd[m + (int64_t)n * ldu] = adam_element(g, mom + m + (int64_t)n * ldm, var + m + (int64_t)n * ldv, s);
  }
};

// ---- kernel ------------------------------------------------------------------------------
// KS_ > 1: KS_ groups of WM_ x WN_ wavefronts share a tile; each group multiplies its own part of
// every K-slab and the groups' accumulators are added through LDS before the epilogue.  For tiles
// so small that a wavefront holds a single accumulator block, this puts two wavefronts on every
// SIMD, so that one's LDS waits hide behind the other's matrix instructions.
// PF_ > 1 (fast path only): that many K-slabs are on their way from memory at any time, held in
// registers until their turn to be stored to LDS.  A tile that runs one workgroup per compute unit
// has nobody to hide a slab's trip from memory behind; with one slab in flight its loop waits for
// memory once per slab.
template <typename T, int BM_, int BN_, int BK_, int WM_, int WN_, int KS_ = 1, int PF_ = 1>
struct GemmTile {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_, KS = KS_, PF = PF_;
  static constexpr int NT = 64 * WM * WN * KS;
  static constexpr int MI = Mfma<T>::MI, KI = Mfma<T>::KI;
  static constexpr int TM = BM / WM / MI, TN = BN / WN / MI;
  static constexpr int VW = Vec16<T>::W;
  static constexpr int PAD = VW;  // keeps rows 16-byte aligned, skews banks for transposed stores
  static constexpr int SA = BM + PAD, SB = BN + PAD;
  static constexpr int NVA = BK * BM / VW / NT, NVB = BK * BN / VW / NT;
  static_assert(BM % (WM * MI) == 0 && BN % (WN * MI) == 0, "wave tiling");
  static_assert(BK % (KI * KS) == 0 && BK % VW == 0, "k tiling");
  static_assert(KS == 1 || (KS - 1) * TM * TN * Mfma<T>::NACC * (NT / KS) <= 2 * BK * (BM + PAD + BN + PAD),
                "the groups' accumulators are exchanged through the operands' LDS buffers");
  static_assert((BK * BM / VW) % NT == 0 && (BK * BN / VW) % NT == 0, "loader tiling");
  static constexpr int LDS_ELEMS = 2 * BK * SA + 2 * BK * SB;  // two buffers of a K-slab of each operand
};

// Which 16-byte piece of a k-contiguous operand slab vector index v handles: KV pieces along k for
// each x.  Sixteen consecutive lanes take sixteen consecutive x at one k piece, the next sixteen
// lanes the next k piece: the transposing LDS stores S[k][x] of 32 lanes then fall into 32 distinct
// banks (with v -> (v / KV, v % KV) two k pieces 2*KV rows apart shared their banks).  Global
// loads do not care: a wavefront's load covers the same set of 64-byte segments either way.
template <int KV>
__device__ __forceinline__ int kcontig_x(int v) {
  return 16 * (v / (16 * KV)) + (v & 15);
}
template <int KV>
__device__ __forceinline__ int kcontig_kv(int v) {
  return (v >> 4) % KV;
}

// Load one K-slab of an operand into registers.  X is the non-K extent (M for A, N for B).
// xcontig: element (x, k) lives at base[x + k*ld]; otherwise at base[k + x*ld].
template <typename T, int BX, int BK, int NT, int NV>
__device__ __forceinline__ void load_slab(T (&reg)[NV][Vec16<T>::W], const T* __restrict__ base, int64_t ld,
                                          int x0, int X, int k0, int kend, bool xcontig, bool vec, int tid,
                                          const int* __restrict__ ksel = nullptr) {
  constexpr int VW = Vec16<T>::W;
  using V = typename Vec16<T>::type;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    int v = tid + i * NT;
    if (xcontig) {
      int k = v / (BX / VW), xv = v % (BX / VW);
      int gx = x0 + xv * VW, gk = k0 + k;
      const int64_t sk = (ksel && gk < kend) ? ksel[gk] : gk;  // stored row of this k
      const T* p = base + gx + sk * ld;
      if (vec) {
        if (gx < X && gk < kend) {
          V t = *reinterpret_cast<const V*>(p);
          const T* tp = reinterpret_cast<const T*>(&t);
#pragma unroll
          for (int e = 0; e < VW; ++e) reg[i][e] = tp[e];
        } else {
#pragma unroll
          for (int e = 0; e < VW; ++e) reg[i][e] = T(0);
        }
      } else {
#pragma unroll
        for (int e = 0; e < VW; ++e) reg[i][e] = (gx + e < X && gk < kend) ? p[e] : T(0);
      }
    } else {
      int x = kcontig_x<BK / VW>(v), kv = kcontig_kv<BK / VW>(v);
      int gx = x0 + x, gk = k0 + kv * VW;
      const T* p = base + gk + (int64_t)gx * ld;
      if (vec) {
        if (gx < X && gk < kend) {
          V t = *reinterpret_cast<const V*>(p);
          const T* tp = reinterpret_cast<const T*>(&t);
#pragma unroll
          for (int e = 0; e < VW; ++e) reg[i][e] = tp[e];
        } else {
#pragma unroll
          for (int e = 0; e < VW; ++e) reg[i][e] = T(0);
        }
      } else {
#pragma unroll
        for (int e = 0; e < VW; ++e) reg[i][e] = (gx < X && gk + e < kend) ? p[e] : T(0);
      }
    }
  }
}

template <typename T, int BX, int BK, int NT, int NV, int STRIDE>
__device__ __forceinline__ void store_slab(T* __restrict__ S, const T (&reg)[NV][Vec16<T>::W], bool xcontig, int tid) {
  constexpr int VW = Vec16<T>::W;
  using V = typename Vec16<T>::type;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    int v = tid + i * NT;
    if (xcontig) {
      int k = v / (BX / VW), xv = v % (BX / VW);
      V t;
      T* tp = reinterpret_cast<T*>(&t);
#pragma unroll
      for (int e = 0; e < VW; ++e) tp[e] = reg[i][e];
      *reinterpret_cast<V*>(S + k * STRIDE + xv * VW) = t;
    } else {
      int x = kcontig_x<BK / VW>(v), kv = kcontig_kv<BK / VW>(v);
#pragma unroll
      for (int e = 0; e < VW; ++e) S[(kv * VW + e) * STRIDE + x] = reg[i][e];
    }
  }
}

// Fast-path loader state: with full tiles, a K extent that is a multiple of the slab and
// 16-byte-aligned operands, every thread walks fixed global pointers (one 16-byte load each,
// bumped by a constant per slab) and fixed LDS offsets; no bounds or layout tests are left in
// the loop and the operand layout is a template constant.
template <typename T, int BX, int BK, int NT, int NV, bool XCONTIG>
struct FastLoader {
  static constexpr int VW = Vec16<T>::W;
  using V = typename Vec16<T>::type;
  const T* ptr[NV];
  int64_t step;
  __device__ __forceinline__ void init(const T* base, int64_t ld, int x0, int k0, int tid) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = tid + i * NT;
      if (XCONTIG) {
        const int k = v / (BX / VW), xv = v % (BX / VW);
        ptr[i] = base + (x0 + xv * VW) + (int64_t)(k0 + k) * ld;
      } else {
        const int x = kcontig_x<BK / VW>(v), kv = kcontig_kv<BK / VW>(v);
        ptr[i] = base + (k0 + kv * VW) + (int64_t)(x0 + x) * ld;
      }
    }
    step = XCONTIG ? (int64_t)BK * ld : (int64_t)BK;
  }
  __device__ __forceinline__ void load(T (&reg)[NV][VW]) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const V t = *reinterpret_cast<const V*>(ptr[i]);
      const T* tp = reinterpret_cast<const T*>(&t);
#pragma unroll
      for (int e = 0; e < VW; ++e) reg[i][e] = tp[e];
      ptr[i] += step;
    }
  }
};

// MODE < 0: general path (any size, alignment and layout, tested at run time).
// MODE in 0..3: fast path, bit 0 = A operand x-contiguous, bit 1 = B operand x-contiguous.
template <typename T, class Cfg, class Epi, int MODE>
__device__ __forceinline__ void gemm_tile_body(const GemmProblem<T>& p, const Epi& epi, const int wg, const int z,
                                               T* __restrict__ smem) {
  using MF = Mfma<T>;
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, NT = Cfg::NT;
  constexpr int MI = Cfg::MI, KI = Cfg::KI, TM = Cfg::TM, TN = Cfg::TN;
  constexpr int SA = Cfg::SA, SB = Cfg::SB, VW = Cfg::VW;
  constexpr bool FAST = MODE >= 0;
  constexpr bool AXC = (MODE & 1) != 0, BXC = (MODE & 2) != 0;

  // (smem: Cfg::LDS_ELEMS elements of the kernel's LDS, 16-byte aligned.  Declared by the kernel, not
  // here: a kernel that holds two instances of this body would otherwise get two arrays.)
  T(*As)[BK * SA] = reinterpret_cast<T(*)[BK * SA]>(smem);
  T(*Bs)[BK * SB] = reinterpret_cast<T(*)[BK * SB]>(smem + 2 * BK * SA);

  // Consecutive workgroup ids are dealt round-robin to the 8 XCDs; give each XCD one
  // contiguous range of tiles so that neighbouring tiles share its L2.
  const int chunk = (p.num_tiles + 7) >> 3;
  const int t = (wg & 7) * chunk + (wg >> 3);
  if (t >= p.num_tiles) return;

  int tm, tn;
  if (p.lower) {
    int bi = (int)((sqrtf(8.0f * (float)t + 1.0f) - 1.0f) * 0.5f);
    while (bi * (bi + 1) / 2 > t) --bi;
    while ((bi + 1) * (bi + 2) / 2 <= t) ++bi;
    tm = bi;
    tn = t - bi * (bi + 1) / 2;
  } else {
    constexpr int GR = SOAPMI_TILE_GROUP_ROWS;
    const int per = GR * p.tiles_n;
    const int g = t / per, r = t - g * per;
    const int rows = min(GR, p.tiles_m - g * GR);
    tm = g * GR + r % rows;
    tn = r / rows;
  }
  const int m0 = tm * BM, n0 = tn * BN;
  const int kbeg = z * p.k_chunk;
  const int kend = min(p.K, kbeg + p.k_chunk);

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  constexpr int KS = Cfg::KS, KSTEPS = BK / KI / KS;  // k steps of a slab per wavefront group
  const int wave_mn = wave % (Cfg::WM * Cfg::WN), wave_k = wave / (Cfg::WM * Cfg::WN);
  const int wm0 = (wave_mn % Cfg::WM) * (TM * MI);
  const int wn0 = (wave_mn / Cfg::WM) * (TN * MI);

  typename MF::Acc acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < MF::NACC; ++r) acc[i][j][r] = T(0);

  T ra[Cfg::NVA][VW], rb[Cfg::NVB][VW];
  const bool a_xc = FAST ? AXC : !p.transA;
  const bool b_xc = FAST ? BXC : (p.transB != 0);
  const int nk = (kend - kbeg + BK - 1) / BK;
  FastLoader<T, BM, BK, NT, Cfg::NVA, AXC> fa;
  FastLoader<T, BN, BK, NT, Cfg::NVB, BXC> fb;

  constexpr int PF = FAST ? Cfg::PF : 1;
  T pa[PF][Cfg::NVA][VW], pb[PF][Cfg::NVB][VW];  // slabs in flight beyond the next one (PF > 1)
  if (nk > 0) {
    if (FAST) {
      fa.init(p.A, p.lda, m0, kbeg, tid);
      fb.init(p.B, p.ldb, n0, kbeg, tid);
      fa.load(ra);
      fb.load(rb);
      if constexpr (PF > 1) {
#pragma unroll
        for (int sl = 1; sl <= PF; ++sl)
          if (sl < nk) {
            fa.load(pa[sl % PF]);
            fb.load(pb[sl % PF]);
          }
      }
    } else {
      load_slab<T, BM, BK, NT, Cfg::NVA>(ra, p.A, p.lda, m0, p.M, kbeg, kend, a_xc, p.vecA, tid);
      load_slab<T, BN, BK, NT, Cfg::NVB>(rb, p.B, p.ldb, n0, p.N, kbeg, kend, b_xc, p.vecB, tid, p.ksel_b);
    }
    store_slab<T, BM, BK, NT, Cfg::NVA, SA>(As[0], ra, a_xc, tid);
    store_slab<T, BN, BK, NT, Cfg::NVB, SB>(Bs[0], rb, b_xc, tid);
  }
  __syncthreads();

  const int krow = lane / MI, idx = lane % MI;
  auto multiply_slab = [&](int buf) {
    const T* as = As[buf];
    const T* bs = Bs[buf];
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk) {
      T fm[TM], fn[TN];
      const int kr = (wave_k * KSTEPS + kk) * KI + krow;
#pragma unroll
      for (int i = 0; i < TM; ++i) fm[i] = as[kr * SA + wm0 + i * MI + idx];
#pragma unroll
      for (int j = 0; j < TN; ++j) fn[j] = bs[kr * SB + wn0 + j * MI + idx];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = MF::mma(fn[j], fm[i], acc[i][j]);
    }
  };
  if constexpr (PF > 1) {
    // Slab kt + 1 waits in register slot (kt + 1) % PF; once it has been stored to LDS the slot takes
    // the load of slab kt + 1 + PF.  The loop is unrolled by PF so that slots are compile-time indices.
    // While slab kt + 1 + PF exists an iteration has no tests in it: a load that is issued only
    // under a condition makes the compiler wait for every load in flight before the next LDS store
    // (it must assume the fewest younger loads), which empties the queue once per slab.
    const int steady = max(0, nk - PF - 1) / PF * PF;
    for (int kt0 = 0; kt0 < steady; kt0 += PF) {
#pragma unroll
      for (int u = 0; u < PF; ++u) {
        const int buf = (kt0 + u) & 1, slot = (u + 1) % PF;
        multiply_slab(buf);
        store_slab<T, BM, BK, NT, Cfg::NVA, SA>(As[buf ^ 1], pa[slot], a_xc, tid);
        store_slab<T, BN, BK, NT, Cfg::NVB, SB>(Bs[buf ^ 1], pb[slot], b_xc, tid);
        fa.load(pa[slot]);
        fb.load(pb[slot]);
        __syncthreads();
      }
    }
    for (int kt0 = steady; kt0 < nk; kt0 += PF) {
#pragma unroll
      for (int u = 0; u < PF; ++u) {
        const int kt = kt0 + u;
        if (kt < nk) {
          const int buf = kt & 1;
          multiply_slab(buf);
          const int slot = (u + 1) % PF;
          if (kt + 1 < nk) {
            store_slab<T, BM, BK, NT, Cfg::NVA, SA>(As[buf ^ 1], pa[slot], a_xc, tid);
            store_slab<T, BN, BK, NT, Cfg::NVB, SB>(Bs[buf ^ 1], pb[slot], b_xc, tid);
          }
          if (kt + 1 + PF < nk) {
            fa.load(pa[slot]);
            fb.load(pb[slot]);
          }
          __syncthreads();
        }
      }
    }
  } else {
    for (int kt = 0; kt < nk; ++kt) {
      const int buf = kt & 1;
      if (kt + 1 < nk) {
        if (FAST) {
          fa.load(ra);
          fb.load(rb);
        } else {
          const int k0 = kbeg + (kt + 1) * BK;
          load_slab<T, BM, BK, NT, Cfg::NVA>(ra, p.A, p.lda, m0, p.M, k0, kend, a_xc, p.vecA, tid);
          load_slab<T, BN, BK, NT, Cfg::NVB>(rb, p.B, p.ldb, n0, p.N, k0, kend, b_xc, p.vecB, tid, p.ksel_b);
        }
      }
      multiply_slab(buf);
      if (kt + 1 < nk) {
        store_slab<T, BM, BK, NT, Cfg::NVA, SA>(As[buf ^ 1], ra, a_xc, tid);
        store_slab<T, BN, BK, NT, Cfg::NVB, SB>(Bs[buf ^ 1], rb, b_xc, tid);
      }
      __syncthreads();
    }
  }

  if constexpr (KS > 1) {
    // (the loop's last barrier is behind every read of the operand buffers)
    constexpr int GT = NT / KS;  // threads of a group
    T* red = smem;
    const int t_in = tid % GT;
    if (wave_k > 0) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int r = 0; r < MF::NACC; ++r)
            red[(((wave_k - 1) * TM + i) * TN + j) * MF::NACC * GT + r * GT + t_in] = acc[i][j][r];
    }
    __syncthreads();
    if (wave_k > 0) return;
#pragma unroll
    for (int g = 1; g < KS; ++g)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int r = 0; r < MF::NACC; ++r)
            acc[i][j][r] += red[(((g - 1) * TM + i) * TN + j) * MF::NACC * GT + r * GT + t_in];
  }

#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + wm0 + i * MI + idx;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int r = 0; r < MF::NACC; ++r) {
        const int n = n0 + wn0 + j * MI + MF::acc_row(r, lane);
        if (FAST || (m < p.M && n < p.N)) epi(m, n, acc[i][j][r], z);
      }
    }
  }
}

template <typename T, class Cfg, class Epi, int MODE>
__global__ __launch_bounds__(Cfg::NT) void gemm_kernel(GemmProblem<T> p, Epi epi) {
  __shared__ __attribute__((aligned(16))) T smem[Cfg::LDS_ELEMS];
  gemm_tile_body<T, Cfg, Epi, MODE>(p, epi, blockIdx.x, blockIdx.y, smem);
}

// Two independent products in one launch: workgroups [0, grid0) take the first problem, the rest
// the second (each with its own operand-layout mode).  Used for the two Gram updates of a step,
// whose tile counts together fill the 256 compute units better than either does alone.
template <typename T, class Cfg, class Epi, int MODE0, int MODE1>
__global__ __launch_bounds__(Cfg::NT) void gemm_pair_kernel(GemmProblem<T> p0, Epi e0, GemmProblem<T> p1, Epi e1,
                                                            int grid0) {
  __shared__ __attribute__((aligned(16))) T smem[Cfg::LDS_ELEMS];
  if ((int)blockIdx.x < grid0) gemm_tile_body<T, Cfg, Epi, MODE0>(p0, e0, blockIdx.x, 0, smem);
  else gemm_tile_body<T, Cfg, Epi, MODE1>(p1, e1, (int)blockIdx.x - grid0, 0, smem);
}

// One problem per blockIdx.z, described in device memory (sizes may be produced by earlier
// kernels of the same stream); workgroups beyond a problem's tile count return at once.
template <typename T>
struct BatchedGemm {
  GemmProblem<T> p;
  EpiStore<T> e;
};
template <typename T, class Cfg>
__global__ __launch_bounds__(Cfg::NT) void gemm_batched_kernel(const BatchedGemm<T>* __restrict__ batch) {
  const BatchedGemm<T> b = batch[blockIdx.z];
  if (b.p.M <= 0 || b.p.N <= 0) return;
  __shared__ __attribute__((aligned(16))) T smem[Cfg::LDS_ELEMS];
  gemm_tile_body<T, Cfg, EpiStore<T>, -1>(b.p, b.e, blockIdx.x, 0, smem);
}

// The same product for blockIdx.z = 0 .. batch-1, with the operands and the result a fixed number of
// elements further on each time (general path: any size and alignment).
template <typename T, class Cfg>
__global__ __launch_bounds__(Cfg::NT) void gemm_strided_kernel(GemmProblem<T> p, EpiStore<T> e, int64_t stride_a,
                                                               int64_t stride_b, int64_t stride_c) {
  p.A += (int64_t)blockIdx.z * stride_a;
  p.B += (int64_t)blockIdx.z * stride_b;
  e.C += (int64_t)blockIdx.z * stride_c;
  __shared__ __attribute__((aligned(16))) T smem[Cfg::LDS_ELEMS];
  gemm_tile_body<T, Cfg, EpiStore<T>, -1>(p, e, blockIdx.x, 0, smem);
}

// Device-side twin of make_problem for the default tile.
template <typename T, class Cfg>
__device__ __forceinline__ void fill_batched(BatchedGemm<T>& b, int transA, int transB, int M, int N, int K,
                                             const T* A, int64_t lda, const T* B, int64_t ldb, T* C, int64_t ldc,
                                             T alpha, T beta) {
  constexpr int VW = Vec16<T>::W;
  b.p.A = A; b.p.B = B; b.p.lda = lda; b.p.ldb = ldb;
  b.p.M = M; b.p.N = N; b.p.K = K;
  b.p.transA = transA; b.p.transB = transB;
  b.p.vecA = ((uintptr_t)A % 16 == 0) && (lda % VW == 0) && ((transA ? K : M) % VW == 0);
  b.p.vecB = ((uintptr_t)B % 16 == 0) && (ldb % VW == 0) && ((transB ? N : K) % VW == 0);
  b.p.tiles_m = (M + Cfg::BM - 1) / Cfg::BM;
  b.p.tiles_n = (N + Cfg::BN - 1) / Cfg::BN;
  b.p.num_tiles = b.p.tiles_m * b.p.tiles_n;
  b.p.lower = 0;
  b.p.ksel_b = nullptr;
  b.p.k_chunk = ((K > 0 ? K : 1) + Cfg::BK - 1) / Cfg::BK * Cfg::BK;
  b.e.C = C; b.e.ldc = ldc; b.e.alpha = alpha; b.e.beta = beta;
}

// Sum split-K partials and apply alpha/beta.
template <typename T>
__global__ void reduce_partials_kernel(const T* __restrict__ part, int splits, int64_t slab, int M, int N, T* C,
                                       int64_t ldc, T alpha, T beta) {
  int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (i >= (int64_t)M * N) return;
  int m = (int)(i % M), n = (int)(i / M);
  T s = T(0);
  for (int z = 0; z < splits; ++z) s += part[(int64_t)z * slab + i];
  T* p = C + m + (int64_t)n * ldc;
  T r = alpha * s;
  if (beta != T(0)) r += beta * (*p);
  *p = r;
}

// ---- host side -----------------------------------------------------------------------------
template <typename T>
struct DefaultTile;
template <>
struct DefaultTile<float> {
  using type = GemmTile<float, 128, 128, 16, 4, 2>;
};
template <>
struct DefaultTile<double> {
  using type = GemmTile<double, 128, 128, 16, 4, 2>;
};

// Tile for products that would give the default tile too few workgroups (1024^2 shapes): four
// wavefronts, 64 x 64.  Measured: 1024^3 fp32 67 TFLOP/s against 28 with the default tile.
template <typename T>
struct SmallTile {
  using type = GemmTile<T, 64, 64, 16, 2, 2>;
};
// fp32: a wavefront's share of the tile is a single 32 x 32 accumulator block, so two groups of four
// wavefronts split each (32 deep) K-slab between them.
template <>
struct SmallTile<float> {
  using type = GemmTile<float, 64, 64, 32, 2, 2, 2, 2>;
};

// True if an M x N output has so few default tiles that the 256 CUs are badly filled: at most half
// a round of workgroups, or a last round under 80 % full within the first four rounds.
template <typename T>
static inline bool prefer_small_tile(int64_t M, int64_t N, bool lower) {
  using Wide = typename DefaultTile<T>::type;
  const int64_t tm = ceil_div64(M, Wide::BM), tn = ceil_div64(N, Wide::BN);
  const int64_t tiles = lower ? tm * (tm + 1) / 2 : tm * tn;
  if (tiles <= 128) return true;
  if (tiles >= 1024) return false;
  const int64_t rounds = ceil_div64(tiles, 256);
  return (double)tiles < 0.8 * (double)(rounds * 256);
}

// Tile for products whose M extent is a panel width (32): tall-skinny block-reflector work.
template <typename T>
struct SkinnyTile;
template <>
struct SkinnyTile<float> {
  using type = GemmTile<float, 32, 128, 32, 1, 4>;
};
template <>
struct SkinnyTile<double> {
  using type = GemmTile<double, 32, 128, 16, 1, 4>;
};

template <typename T>
static inline bool vec_ok(const T* p, int64_t ld, int contig_extent) {
  constexpr int VW = Vec16<T>::W;
  return (reinterpret_cast<uintptr_t>(p) % 16 == 0) && (ld % VW == 0) && (contig_extent % VW == 0);
}

template <typename T, class Cfg = typename DefaultTile<T>::type>
static inline GemmProblem<T> make_problem(int transA, int transB, int M, int N, int K, const T* A, int64_t lda,
                                          const T* B, int64_t ldb, bool lower) {
  GemmProblem<T> p;
  p.A = A; p.B = B; p.lda = lda; p.ldb = ldb;
  p.M = M; p.N = N; p.K = K;
  p.transA = transA; p.transB = transB;
  // contiguous extent: A not transposed -> m, transposed -> k ; B not transposed -> k, transposed -> n
  p.vecA = vec_ok(A, lda, transA ? K : M);
  p.vecB = vec_ok(B, ldb, transB ? N : K);
  p.tiles_m = (int)ceil_div64(M, Cfg::BM);
  p.tiles_n = (int)ceil_div64(N, Cfg::BN);
  p.lower = lower ? 1 : 0;
  p.ksel_b = nullptr;
  p.num_tiles = lower ? p.tiles_m * (p.tiles_m + 1) / 2 : p.tiles_m * p.tiles_n;
  p.k_chunk = (int)(ceil_div64(K > 0 ? K : 1, Cfg::BK) * Cfg::BK);
  return p;
}

template <typename T, class Epi, class Cfg = typename DefaultTile<T>::type>
static inline int launch_gemm(hipStream_t stream, const GemmProblem<T>& p, const Epi& epi, int k_splits = 1) {
  if (p.M <= 0 || p.N <= 0) return kOk;
  const int chunk = (p.num_tiles + 7) / 8;
  dim3 grid(8 * chunk, k_splits, 1);
  // (K slices start at multiples of k_chunk, so with K and k_chunk multiples of the slab every
  // slice, a shorter last one included, is a whole number of slabs)
  const bool fast = p.vecA && p.vecB && p.M % Cfg::BM == 0 && p.N % Cfg::BN == 0 && p.K > 0 &&
                    p.K % Cfg::BK == 0 && p.k_chunk % Cfg::BK == 0;
  const int mode = fast ? ((p.transA ? 0 : 1) | (p.transB ? 2 : 0)) : -1;
  switch (mode) {
    case 0: hipLaunchKernelGGL((gemm_kernel<T, Cfg, Epi, 0>), grid, dim3(Cfg::NT), 0, stream, p, epi); break;
    case 1: hipLaunchKernelGGL((gemm_kernel<T, Cfg, Epi, 1>), grid, dim3(Cfg::NT), 0, stream, p, epi); break;
    case 2: hipLaunchKernelGGL((gemm_kernel<T, Cfg, Epi, 2>), grid, dim3(Cfg::NT), 0, stream, p, epi); break;
    case 3: hipLaunchKernelGGL((gemm_kernel<T, Cfg, Epi, 3>), grid, dim3(Cfg::NT), 0, stream, p, epi); break;
    default: hipLaunchKernelGGL((gemm_kernel<T, Cfg, Epi, -1>), grid, dim3(Cfg::NT), 0, stream, p, epi); break;
  }
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

// Fast-path mode of a problem for tile Cfg (see launch_gemm), or -1.
template <typename T, class Cfg>
static inline int fast_mode(const GemmProblem<T>& p) {
  const bool fast = p.vecA && p.vecB && p.M % Cfg::BM == 0 && p.N % Cfg::BN == 0 && p.K > 0 && p.K % Cfg::BK == 0 &&
                    p.k_chunk % Cfg::BK == 0;
  return fast ? ((p.transA ? 0 : 1) | (p.transB ? 2 : 0)) : -1;
}

// Launches two problems (same tile, same epilogue type) as one grid when their mode pair is one of
// those compiled: (0, 3), (3, 0) -- the two Gram products of one gradient -- or both general.
// Returns false without launching anything otherwise.
template <typename T, class Epi, class Cfg>
static inline bool launch_gemm_pair(hipStream_t stream, const GemmProblem<T>& p0, const Epi& e0,
                                    const GemmProblem<T>& p1, const Epi& e1, int* rc) {
  *rc = kOk;
  if (p0.M <= 0 || p0.N <= 0 || p1.M <= 0 || p1.N <= 0) return false;
  const int m0 = fast_mode<T, Cfg>(p0), m1 = fast_mode<T, Cfg>(p1);
  const int grid0 = 8 * ((p0.num_tiles + 7) / 8), grid1 = 8 * ((p1.num_tiles + 7) / 8);
  const dim3 grid(grid0 + grid1);
  if (m0 == 0 && m1 == 3)
    hipLaunchKernelGGL((gemm_pair_kernel<T, Cfg, Epi, 0, 3>), grid, dim3(Cfg::NT), 0, stream, p0, e0, p1, e1, grid0);
  else if (m0 == 3 && m1 == 0)
    hipLaunchKernelGGL((gemm_pair_kernel<T, Cfg, Epi, 3, 0>), grid, dim3(Cfg::NT), 0, stream, p0, e0, p1, e1, grid0);
  else if (m0 == -1 && m1 == -1)
    hipLaunchKernelGGL((gemm_pair_kernel<T, Cfg, Epi, -1, -1>), grid, dim3(Cfg::NT), 0, stream, p0, e0, p1, e1, grid0);
  else
    return false;
  if (hipGetLastError() != hipSuccess) {
    set_error("kernel launch failed");
    *rc = kRuntimeError;
  }
  return true;
}

// C = alpha*op(A)*op(B) + beta*C.  If `partials` is non-null and k_splits > 1 the K range is
// cut into k_splits slices whose partial products are summed by a second kernel (fixed
// order, so the result does not depend on scheduling).
template <typename T, class Cfg = typename DefaultTile<T>::type>
static inline int gemm(hipStream_t stream, int transA, int transB, int M, int N, int K, T alpha, const T* A,
                       int64_t lda, const T* B, int64_t ldb, T beta, T* C, int64_t ldc, int k_splits = 1,
                       T* partials = nullptr) {
  if (M <= 0 || N <= 0) return kOk;
  if constexpr (std::is_same<Cfg, typename DefaultTile<T>::type>::value) {
    if (k_splits <= 1 && prefer_small_tile<T>(M, N, false))
      return gemm<T, typename SmallTile<T>::type>(stream, transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
  }
  GemmProblem<T> p = make_problem<T, Cfg>(transA, transB, M, N, K, A, lda, B, ldb, false);
  if (k_splits > 1 && partials != nullptr && K > Cfg::BK) {
    int64_t slabs = ceil_div64(K, Cfg::BK);
    p.k_chunk = (int)(ceil_div64(slabs, k_splits) * Cfg::BK);
    int splits = (int)ceil_div64(K, p.k_chunk);
    EpiPartial<T> ep{partials, (int64_t)M, (int64_t)M * N};
    int rc = launch_gemm<T, EpiPartial<T>, Cfg>(stream, p, ep, splits);
    if (rc) return rc;
    int64_t total = (int64_t)M * N;
    hipLaunchKernelGGL((reduce_partials_kernel<T>), dim3((unsigned)ceil_div64(total, 256)), dim3(256), 0, stream,
                       partials, splits, (int64_t)M * N, M, N, C, ldc, alpha, beta);
    SOAPMI_LAUNCH_CHECK();
    return kOk;
  }
  EpiStore<T> ep{C, ldc, alpha, beta};
  return launch_gemm<T, EpiStore<T>, Cfg>(stream, p, ep, 1);
}

// C_b = alpha * A_b * B_b + beta * C_b for b = 0 .. batch-1 in one launch (no transposes); operand b
// starts b * stride elements after operand 0.
template <typename T, class Cfg>
static inline int gemm_strided_batch(hipStream_t stream, int M, int N, int K, T alpha, const T* A, int64_t lda,
                                     int64_t stride_a, const T* B, int64_t ldb, int64_t stride_b, T beta, T* C,
                                     int64_t ldc, int64_t stride_c, int batch) {
  if (M <= 0 || N <= 0 || batch <= 0) return kOk;
  constexpr int VW = Vec16<T>::W;
  GemmProblem<T> p = make_problem<T, Cfg>(0, 0, M, N, K, A, lda, B, ldb, false);
  p.vecA = p.vecA && stride_a % VW == 0;
  p.vecB = p.vecB && stride_b % VW == 0;
  EpiStore<T> ep{C, ldc, alpha, beta};
  const int chunk = (p.num_tiles + 7) / 8;
  hipLaunchKernelGGL((gemm_strided_kernel<T, Cfg>), dim3(8 * chunk, 1, batch), dim3(Cfg::NT), 0, stream, p, ep, stride_a,
                     stride_b, stride_c);
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

// op(A) op(B) cut into K slices whose partial products stay unreduced in `partials` (slice z at
// partials + z * M * N, column-major with leading dimension M), for consumers that sum the slices
// themselves.  *splits_out receives the number of slices written (at least 1).
template <typename T, class Cfg = typename DefaultTile<T>::type>
static inline int gemm_to_partials(hipStream_t stream, int transA, int transB, int M, int N, int K, const T* A,
                                   int64_t lda, const T* B, int64_t ldb, int k_splits, T* partials, int* splits_out) {
  *splits_out = 1;
  if (M <= 0 || N <= 0) return kOk;
  GemmProblem<T> p = make_problem<T, Cfg>(transA, transB, M, N, K, A, lda, B, ldb, false);
  int splits = 1;
  if (k_splits > 1 && K > Cfg::BK) {
    const int64_t slabs = ceil_div64(K, Cfg::BK);
    p.k_chunk = (int)(ceil_div64(slabs, k_splits) * Cfg::BK);
    splits = (int)ceil_div64(K, p.k_chunk);
  }
  *splits_out = splits;
  EpiPartial<T> ep{partials, (int64_t)M, (int64_t)M * N};
  return launch_gemm<T, EpiPartial<T>, Cfg>(stream, p, ep, splits);
}

// Square product restricted to the tiles on or below the diagonal of C (n x n): entries of C above
// the diagonal tiles are neither read nor written; inside diagonal tiles the whole tile is updated.
template <typename T, class Cfg = typename DefaultTile<T>::type>
static inline int gemm_lower(hipStream_t stream, int transA, int transB, int n, int K, T alpha, const T* A,
                             int64_t lda, const T* B, int64_t ldb, T beta, T* C, int64_t ldc) {
  if (n <= 0) return kOk;
  GemmProblem<T> p = make_problem<T, Cfg>(transA, transB, n, n, K, A, lda, B, ldb, true);
  EpiStore<T> ep{C, ldc, alpha, beta};
  return launch_gemm<T, EpiStore<T>, Cfg>(stream, p, ep, 1);
}

}  // namespace soapmi
