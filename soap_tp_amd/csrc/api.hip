// extern "C" surface of libsoap_mi355.so (declared in include/soap_mi355.h).
#include <stdarg.h>

#include <atomic>
#include <condition_variable>
#include <mutex>

#include "../../include/soap_mi355.h"
#include "common.hpp"
#include "eigh.hpp"
#include "elementwise.hpp"
#include "gemm.hpp"
#include "qr.hpp"
#include "refresh.hpp"

namespace soapmi {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
const char* last_error() { return g_error; }

// Per-device grow-only scratch used when the caller passes no workspace.
struct InternalScratch {
  void* ptr = nullptr;
  size_t size = 0;
};
static InternalScratch g_scratch[64];
// largest grid for which the QR panel runs as one persistent launch (see soapmi_set_option)
static std::atomic<int> g_qr_persistent_max_wg{kQrPersistentMaxWg};
// polls a workgroup spends waiting for another one's message before it gives up (see soapmi_set_option)
static std::atomic<unsigned> g_message_spin_limit{kQrSpinLimit};
// panel columns the QR factors per message round (see soapmi_set_option)
static std::atomic<int> g_qr_columns_per_round{kQrWholePanel};
// streams a basis refresh uses: 2 = the two factorisation chains side by side, 1 = one after the other
static std::atomic<int> g_refresh_streams{2};
// 1 = a QR panel's in-block update rides along in the next panel's launch, 0 = a launch of its own
static std::atomic<int> g_qr_carry_update{1};
// widest compact-WY reflector of the QR: kQrSuper = three blocking levels, kBrMax = two, 0 = by size
static std::atomic<int> g_qr_super_block{0};
// tridiagonalisation of the eigensolver: kEighOneStage or kEighTwoStage (see soapmi_set_option)
static std::atomic<int> g_eigh_algorithm{kEighOneStage};
static std::mutex g_scratch_mutex;

static int resolve_workspace(void* user, size_t user_bytes, size_t need, void** out) {
  if (user != nullptr) {
    if (user_bytes < need) {
      set_error("workspace holds %zu bytes, %zu are required", user_bytes, need);
      return kWorkspaceTooSmall;
    }
    *out = user;
    return kOk;
  }
  int dev = 0;
  SOAPMI_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) {
    set_error("unsupported device index %d", dev);
    return kRuntimeError;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  InternalScratch& s = g_scratch[dev];
  if (s.size < need) {
    if (s.ptr) {
      SOAPMI_HIP(hipDeviceSynchronize());
      SOAPMI_HIP(hipFree(s.ptr));
      s.ptr = nullptr;
      s.size = 0;
    }
    SOAPMI_HIP(hipMalloc(&s.ptr, need));
    s.size = need;
  }
  *out = s.ptr;
  return kOk;
}

// A second stream per device (default priority) and two events, created on first use and kept
// for the life of the process: the basis refresh runs its two independent factorisation chains
// side by side, forked from and joined back into the caller's stream with events, so the caller
// still sees everything ordered on the stream it passed.
struct SideStream {
  hipStream_t stream = nullptr;
  hipEvent_t fork = nullptr;
  hipEvent_t join = nullptr;
};
static SideStream g_side[64];

static int side_stream(SideStream** out) {
  int dev = 0;
  SOAPMI_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) {
    set_error("unsupported device index %d", dev);
    return kRuntimeError;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  SideStream& side = g_side[dev];
  if (!side.stream) {
    SOAPMI_HIP(hipStreamCreateWithFlags(&side.stream, hipStreamNonBlocking));
    SOAPMI_HIP(hipEventCreateWithFlags(&side.fork, hipEventDisableTiming));
    SOAPMI_HIP(hipEventCreateWithFlags(&side.join, hipEventDisableTiming));
  }
  *out = &side;
  return kOk;
}

// One word of pinned host memory per device that the factorisations' last kernel raises when a
// persistent kernel gave up waiting for a message (the output is NaN-poisoned then).  The host reads
// it without synchronising: soapmi_device_error_flag.
static int* g_report[64];

static int device_report(int** out) {
  int dev = 0;
  SOAPMI_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) {
    set_error("unsupported device index %d", dev);
    return kRuntimeError;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_report[dev]) {
    void* p = nullptr;
    SOAPMI_HIP(hipHostMalloc(&p, 64, hipHostMallocDefault));
    memset(p, 0, 64);
    g_report[dev] = static_cast<int*>(p);
  }
  *out = g_report[dev];
  return kOk;
}

// A caller-owned status word (device-writable memory: device memory or pinned host memory) that the
// factorisations enqueued by the calling thread raise instead of the per-device report word, so that
// a failure can be told apart per optimizer state: soapmi_set_status_word.
static thread_local int* t_status_word = nullptr;

// Where a factorisation's last kernel reports a failure: the caller's status word if one is set for
// this thread, else the device's report word.
static int failure_report(int** out) {
  if (t_status_word) {
    *out = t_status_word;
    return kOk;
  }
  return device_report(out);
}

// Persistent kernels (the QR panel kernel, the tridiagonalisation's column kernel) wait inside the
// kernel for messages from the other workgroups of their launch, so all workgroups of a launch must
// be resident together.  One launch always is (at most 128 workgroups on 256 compute units), but
// several factorisations running side by side on different streams could each hold part of the
// chip while waiting for workgroups that find no free slot.  The library therefore keeps, per
// device, the workgroup counts of the factorisations that may still be running (an event marks the
// end of each) and makes a new one wait, on the device, for earlier ones until the sum fits the
// budget.  Nothing here synchronises the host with the device; host threads that enqueue
// factorisations at the same time only share the bookkeeping.
static std::atomic<int> g_persistent_budget{256};

// Compute units of the current device (looked up once per device): a persistent workgroup of the
// panel kernels takes a whole one, so neither the budget nor one launch may exceed their number on
// a partitioned or masked device.
static int compute_unit_count() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int count = cached[dev].load();
  if (count == 0) {
    if (hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || count <= 0) count = 256;
    cached[dev].store(count);
  }
  return count;
}

struct PersistentLease {
  hipEvent_t done = nullptr;
  int workgroups = 0;
  bool active = false;    // taken by a factorisation that may still be running
  bool recorded = false;  // its end has been recorded in `done` (false while its launches are still being enqueued)
};
struct PersistentLedger {
  std::mutex mutex;               // guards the leases; held for the bookkeeping only, not while launching
  std::condition_variable changed;  // a lease was recorded or given up
  PersistentLease leases[32];
};
static PersistentLedger g_ledger[64];

class PersistentGuard {
 public:
  PersistentGuard() = default;
  PersistentGuard(const PersistentGuard&) = delete;
  PersistentGuard& operator=(const PersistentGuard&) = delete;
  ~PersistentGuard() {
    if (ledger_ && lease_) {  // left without release(): nothing was recorded
      std::lock_guard<std::mutex> lock(ledger_->mutex);
      lease_->active = false;
      ledger_->changed.notify_all();
    }
  }
  // Call before the first launch of a factorisation whose persistent kernels have up to `workgroups`
  // workgroups, on the stream it will run on.  Threads may enqueue factorisations side by side: one
  // that has to wait for a factorisation another thread is still enqueueing waits on the host until
  // that one's end has been recorded, then on the device for the recorded event.
  int acquire(hipStream_t stream, int workgroups) {
    int dev = 0;
    SOAPMI_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64) {
      set_error("unsupported device index %d", dev);
      return kRuntimeError;
    }
    ledger_ = &g_ledger[dev];
    stream_ = stream;
    const int budget = std::min(g_persistent_budget.load(), compute_unit_count());
    std::unique_lock<std::mutex> lock(ledger_->mutex);
    int held = workgroups;
    for (;;) {
      int in_flight = 0;
      PersistentLease* free_slot = nullptr;
      for (PersistentLease& lease : ledger_->leases) {
        if (lease.active && lease.recorded && hipEventQuery(lease.done) == hipSuccess) lease.active = false;
        if (lease.active) in_flight += lease.workgroups;
        else if (!free_slot) free_slot = &lease;
      }
      (void)hipGetLastError();  // hipEventQuery reports "not ready" through the error state
      if ((in_flight + held <= budget || in_flight == 0) && free_slot) {  // (one larger than the budget runs alone)
        lease_ = free_slot;
        break;
      }
      // Wait for one earlier factorisation and look again.  A factorisation this one waits for never
      // runs beside it, so the two together hold at most the larger of their counts at any time: the
      // waited-for entry is folded into this one.
      PersistentLease* recorded = nullptr;
      for (PersistentLease& lease : ledger_->leases)
        if (lease.active && lease.recorded) {
          recorded = &lease;
          break;
        }
      if (recorded) {
        SOAPMI_HIP(hipStreamWaitEvent(stream, recorded->done, 0));
        if (recorded->workgroups > held) held = recorded->workgroups;
        recorded->active = false;
      } else {
        ledger_->changed.wait(lock);  // every active one is still being enqueued by another thread
      }
    }
    if (!lease_->done) SOAPMI_HIP(hipEventCreateWithFlags(&lease_->done, hipEventDisableTiming));
    lease_->workgroups = held;
    lease_->active = true;
    lease_->recorded = false;
    return kOk;
  }
  // Call after the last launch of the factorisation.
  int release() {
    if (!lease_) return kOk;
    PersistentLease* lease = lease_;
    lease_ = nullptr;
    hipError_t e = hipEventRecord(lease->done, stream_);
    std::lock_guard<std::mutex> lock(ledger_->mutex);
    if (e != hipSuccess) {
      lease->active = false;
      ledger_->changed.notify_all();
      set_error("hipEventRecord failed: %s", hipGetErrorString(e));
      return kRuntimeError;
    }
    lease->recorded = true;
    ledger_->changed.notify_all();
    return kOk;
  }

 private:
  PersistentLedger* ledger_ = nullptr;
  PersistentLease* lease_ = nullptr;
  hipStream_t stream_ = nullptr;
};

// Device memory for the entry point that allocates nothing: two rows x cols temporaries of at most
// kStaticScratchElements floats each (32 MiB in all), part of the code object, so every device
// the library runs on holds its own copy from module load to process exit.  In host code the
// array's name is only a handle for hipGetSymbolAddress: the address of this device's copy is
// looked up once per device and that pointer is what kernels receive.
constexpr int64_t kStaticScratchElements = 4194304;
static __device__ __align__(256) float scratch[2 * kStaticScratchElements];
static float* g_static_scratch[64];

static int static_scratch_address(float** out) {
  int dev = 0;
  SOAPMI_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) {
    set_error("unsupported device index %d", dev);
    return kRuntimeError;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_static_scratch[dev]) {
    void* address = nullptr;
    SOAPMI_HIP(hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)));
    if (!address) {
      set_error("hipGetSymbolAddress returned a null address for the static scratch");
      return kRuntimeError;
    }
    g_static_scratch[dev] = static_cast<float*>(address);
  }
  *out = g_static_scratch[dev];
  return kOk;
}

static AdamScalars make_adam_scalars(int64_t step, double beta1, double beta2, double eps_in) {
  AdamScalars s;
  s.beta1 = (float)beta1;
  s.beta2 = (float)beta2;
  s.one_minus_beta1 = (float)(1.0 - beta1);
  s.one_minus_beta2 = (float)(1.0 - beta2);
  s.bias_correction1 = (float)(1.0 - pow(beta1, (double)step));
  s.sqrt_bias_correction2 = (float)sqrt(1.0 - pow(beta2, (double)step));
  s.eps = (float)eps_in;
  return s;
}

static int check_adam_args(int64_t step, double beta1, double beta2, double eps) {
  SOAPMI_REQUIRE(step >= 1, "step must be positive, got %lld.", (long long)step);
  SOAPMI_REQUIRE(beta1 >= 0.0 && beta1 < 1.0, "beta1 must be in [0, 1), got %g.", beta1);
  SOAPMI_REQUIRE(beta2 >= 0.0 && beta2 < 1.0, "beta2 must be in [0, 1), got %g.", beta2);
  SOAPMI_REQUIRE(eps > 0.0, "eps must be positive, got %g.", eps);
  return kOk;
}

}  // namespace soapmi

using namespace soapmi;

// Workspace of an eigensolve whichever tridiagonalisation is selected when the call is made: the
// option can change between a caller's size query and its call.
template <typename T>
static size_t eigh_workspace_bytes_any(int64_t n) {
  return std::max(eigh_workspace_bytes<T>(n, kEighOneStage), eigh_workspace_bytes<T>(n, kEighTwoStage));
}

template <typename T>
static int eigh_entry(T* a, T* eigenvalues, T* q, int64_t n, int64_t lda, int64_t ldq, void* workspace,
                      size_t workspace_bytes, void* stream) {
  SOAPMI_REQUIRE(a && eigenvalues && q, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(n > 0, "matrix dimensions and block size must be positive");
  SOAPMI_REQUIRE(lda >= n && ldq >= n, "leading dimensions are too small");
  SOAPMI_REQUIRE(n <= 32768, "matrix size %lld exceeds the supported maximum 32768", (long long)n);
  const int algorithm = g_eigh_algorithm.load();  // (read once: everything below uses this value)
  const size_t need = eigh_workspace_bytes<T>(n, algorithm);
  void* ws = nullptr;
  int rc = resolve_workspace(workspace, workspace_bytes, need, &ws);
  if (rc) return rc;
  Workspace w(ws, need);
  EighWorkspace<T> ews;
  eigh_workspace_layout<T>(w, n, &ews, algorithm);
  int* report = nullptr;
  rc = failure_report(&report);
  if (rc) return rc;
  PersistentGuard guard;
  rc = guard.acquire((hipStream_t)stream, (int)ceil_div64(n, 256));
  if (rc) return rc;
  rc = eigh_ascending<T>((hipStream_t)stream, a, lda, eigenvalues, q, ldq, (int)n, ews, g_message_spin_limit.load(),
                         report, algorithm);
  const int rc_release = guard.release();
  return rc ? rc : rc_release;
}

extern "C" {

const char* soapmi_compiled_gpu_backend(void) { return "rocm"; }

void soapmi_world_rank_and_size(int* rank, int* size) {
  if (rank) *rank = 0;
  if (size) *size = 1;
}

const char* soapmi_last_error(void) { return last_error(); }

int soapmi_device_error_flag(int clear) {
  int* report = nullptr;
  int rc = device_report(&report);
  if (rc) return rc;
  // (one exchange: a kernel that raises the word between a read and a separate clearing store would be lost)
  const int value = clear ? __atomic_exchange_n(report, 0, __ATOMIC_ACQ_REL) : __atomic_load_n(report, __ATOMIC_ACQUIRE);
  return value != 0 ? 1 : 0;
}

int soapmi_set_status_word(int* word) {
  t_status_word = word;
  return kOk;
}

int soapmi_set_option(const char* name, int64_t value) {
  SOAPMI_REQUIRE(name, "option name must not be null");
  if (strcmp(name, "qr_persistent_max_workgroups") == 0) {
    SOAPMI_REQUIRE(value >= 0 && value <= kQrPersistentMaxWg, "qr_persistent_max_workgroups must be in 0..%d",
                   kQrPersistentMaxWg);
    g_qr_persistent_max_wg.store((int)value);
    return kOk;
  }
  if (strcmp(name, "qr_columns_per_round") == 0) {
    SOAPMI_REQUIRE((value >= 1 && value <= kQrRoundMax) || value == kQrWholePanel,
                   "qr_columns_per_round must be in 1..%d or %d (the whole panel)", kQrRoundMax, kQrWholePanel);
    g_qr_columns_per_round.store((int)value);
    return kOk;
  }
  if (strcmp(name, "message_spin_limit") == 0) {
    SOAPMI_REQUIRE(value >= 0 && value <= (int64_t)kQrSpinLimit, "message_spin_limit must be in 0..%u", kQrSpinLimit);
    g_message_spin_limit.store((unsigned)value);
    return kOk;
  }
  if (strcmp(name, "persistent_workgroup_budget") == 0) {
    SOAPMI_REQUIRE(value >= 1 && value <= 256, "persistent_workgroup_budget must be in 1..256");
    g_persistent_budget.store((int)value);
    return kOk;
  }
  if (strcmp(name, "eigh_algorithm") == 0) {
    SOAPMI_REQUIRE(value == kEighOneStage || value == kEighTwoStage, "eigh_algorithm must be 1 (one-stage) or 2 (two-stage)");
    g_eigh_algorithm.store((int)value);
    return kOk;
  }
  if (strcmp(name, "qr_carry_update") == 0) {
    SOAPMI_REQUIRE(value == 0 || value == 1, "qr_carry_update must be 0 or 1");
    g_qr_carry_update.store((int)value);
    return kOk;
  }
  if (strcmp(name, "qr_super_block") == 0) {
    SOAPMI_REQUIRE(value == 0 || value == kBrMax || value == kQrSuper, "qr_super_block must be 0, %d or %d", kBrMax,
                   kQrSuper);
    g_qr_super_block.store((int)value);
    return kOk;
  }
  if (strcmp(name, "refresh_streams") == 0) {
    SOAPMI_REQUIRE(value == 1 || value == 2, "refresh_streams must be 1 or 2");
    g_refresh_streams.store((int)value);
    return kOk;
  }
  set_error("unknown option '%s'", name);
  return kInvalidArgument;
}

int soapmi_gemm_f32(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha, const float* a,
                    int64_t lda, const float* b, int64_t ldb, float beta, float* c, int64_t ldc, void* stream) {
  SOAPMI_REQUIRE(m >= 0 && n >= 0 && k >= 0, "matrix dimensions must be non-negative");
  SOAPMI_REQUIRE(a && b && c, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(lda >= (trans_a ? k : m) && ldb >= (trans_b ? n : k) && ldc >= m && lda > 0 && ldb > 0 && ldc > 0,
                 "leading dimensions are too small");
  return gemm<float>((hipStream_t)stream, trans_a, trans_b, (int)m, (int)n, (int)k, alpha, a, lda, b, ldb, beta, c,
                     ldc);
}

int soapmi_gemm_f64(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, double alpha, const double* a,
                    int64_t lda, const double* b, int64_t ldb, double beta, double* c, int64_t ldc, void* stream) {
  SOAPMI_REQUIRE(m >= 0 && n >= 0 && k >= 0, "matrix dimensions must be non-negative");
  SOAPMI_REQUIRE(a && b && c, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(lda >= (trans_a ? k : m) && ldb >= (trans_b ? n : k) && ldc >= m && lda > 0 && ldb > 0 && ldc > 0,
                 "leading dimensions are too small");
  return gemm<double>((hipStream_t)stream, trans_a, trans_b, (int)m, (int)n, (int)k, alpha, a, lda, b, ldb, beta,
                      c, ldc);
}

int soapmi_gram_ema_f32(const float* g, int64_t rows, int64_t cols, int64_t ldg, int g_row_major, int side,
                        float* p, int64_t ldp, float beta, int mirror, void* stream) {
  SOAPMI_REQUIRE(g && p, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(rows >= 0 && cols >= 0, "matrix dimensions must be non-negative");
  SOAPMI_REQUIRE(side == 0 || side == 1, "side must be 0 (left) or 1 (right), got %d.", side);
  SOAPMI_REQUIRE(beta >= 0.0f && beta <= 1.0f, "beta must be in [0, 1], got %g.", (double)beta);
  SOAPMI_REQUIRE(ldg >= (g_row_major ? cols : rows) && ldg > 0, "gradient leading dimension is too small");
  const int64_t n = side == 0 ? rows : cols;
  const int64_t k = side == 0 ? cols : rows;
  SOAPMI_REQUIRE(ldp >= n && ldp > 0, "preconditioner leading dimension is too small");
  if (n == 0) return kOk;
  // Stored matrix S (column-major, ld = ldg): row-major G is S = G^T (cols x rows).
  // left  = G G^T : row-major -> S^T S (transA=1, transB=0) ; col-major -> S S^T (0, 1)
  // right = G^T G : row-major -> S S^T (0, 1)               ; col-major -> S^T S (1, 0)
  const bool stts = (side == 0) == (g_row_major != 0);
  const int ta = stts ? 1 : 0, tb = stts ? 0 : 1;
  EpiEmaLower<float> epi{p, ldp, 1.0f - beta, mirror};
  if (prefer_small_tile<float>(n, n, true)) {
    using Small = SmallTile<float>::type;
    GemmProblem<float> prob = make_problem<float, Small>(ta, tb, (int)n, (int)n, (int)k, g, ldg, g, ldg, true);
    return launch_gemm<float, EpiEmaLower<float>, Small>((hipStream_t)stream, prob, epi, 1);
  }
  GemmProblem<float> prob = make_problem<float>(ta, tb, (int)n, (int)n, (int)k, g, ldg, g, ldg, true);
  return launch_gemm<float>((hipStream_t)stream, prob, epi, 1);
}

int soapmi_gram_ema_pair_f32(const float* g, int64_t rows, int64_t cols, int64_t ldg, int g_row_major, float* left,
                             int64_t ldl, float* right, int64_t ldr, float beta, int mirror, void* stream) {
  SOAPMI_REQUIRE(g && left && right, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(rows > 0 && cols > 0, "matrix dimensions must be positive");
  SOAPMI_REQUIRE(beta >= 0.0f && beta <= 1.0f, "beta must be in [0, 1], got %g.", (double)beta);
  SOAPMI_REQUIRE(ldg >= (g_row_major ? cols : rows) && ldg > 0, "gradient leading dimension is too small");
  SOAPMI_REQUIRE(ldl >= rows && ldr >= cols, "preconditioner leading dimension is too small");
  SOAPMI_REQUIRE(left != right, "the two preconditioners must not overlap");
  // see soapmi_gram_ema_f32 for the operand transposes of each side
  const int lta = g_row_major ? 1 : 0, ltb = g_row_major ? 0 : 1;
  const int rta = ltb, rtb = lta;
  EpiEmaLower<float> el{left, ldl, 1.0f - beta, mirror}, er{right, ldr, 1.0f - beta, mirror};
  using Wide = DefaultTile<float>::type;
  using Small = SmallTile<float>::type;
  const int64_t tl = ceil_div64(rows, Wide::BM), tr = ceil_div64(cols, Wide::BM);
  const int64_t tiles = tl * (tl + 1) / 2 + tr * (tr + 1) / 2;  // default tiles of both lower triangles together
  // the 64 x 64 tile when the default one would fill the compute units badly: few tiles, or a last
  // round of workgroups that is mostly empty (4096^2: 1056 tiles, a fifth round with 32 of 256)
  bool small = tiles <= 128;
  if (!small && tiles < 2048) small = (double)tiles < 0.85 * (double)(ceil_div64(tiles, 256) * 256);
  int rc = kOk;
  bool launched;
  if (small) {
    GemmProblem<float> pl = make_problem<float, Small>(lta, ltb, (int)rows, (int)rows, (int)cols, g, ldg, g, ldg, true);
    GemmProblem<float> pr = make_problem<float, Small>(rta, rtb, (int)cols, (int)cols, (int)rows, g, ldg, g, ldg, true);
    launched = launch_gemm_pair<float, EpiEmaLower<float>, Small>((hipStream_t)stream, pl, el, pr, er, &rc);
  } else {
    GemmProblem<float> pl = make_problem<float, Wide>(lta, ltb, (int)rows, (int)rows, (int)cols, g, ldg, g, ldg, true);
    GemmProblem<float> pr = make_problem<float, Wide>(rta, rtb, (int)cols, (int)cols, (int)rows, g, ldg, g, ldg, true);
    launched = launch_gemm_pair<float, EpiEmaLower<float>, Wide>((hipStream_t)stream, pl, el, pr, er, &rc);
  }
  if (launched) return rc;
  // a layout pair that has no joint kernel: one launch per side
  rc = soapmi_gram_ema_f32(g, rows, cols, ldg, g_row_major, 0, left, ldl, beta, mirror, stream);
  if (rc) return rc;
  return soapmi_gram_ema_f32(g, rows, cols, ldg, g_row_major, 1, right, ldr, beta, mirror, stream);
}

int soapmi_symmetrize_lower_f32(float* p, int64_t n, int64_t ldp, void* stream) {
  SOAPMI_REQUIRE(p, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(n >= 0 && ldp >= n && ldp > 0, "invalid matrix size or leading dimension");
  if (n == 0) return kOk;
  unsigned nb = (unsigned)ceil_div64(n, 64);
  hipLaunchKernelGGL((symmetrize_lower_kernel<float>), dim3(nb, nb), dim3(256), 0, (hipStream_t)stream, p, ldp,
                     (int)n);
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

size_t soapmi_rotate_workspace_bytes(int64_t rows, int64_t cols) {
  WorkspaceSizer w;
  w.take<float>((size_t)rows * cols);
  return w.total();
}

int soapmi_rotate_f32(const float* ql, float* x, const float* qr, int64_t rows, int64_t cols, int64_t ldql,
                      int64_t ldx, int64_t ldqr, int forward, void* workspace, size_t workspace_bytes,
                      void* stream) {
  SOAPMI_REQUIRE(ql && x && qr, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(rows > 0 && cols > 0 && ldql > 0 && ldx > 0 && ldqr > 0,
                 "matrix dimensions and leading dimensions must be positive");
  SOAPMI_REQUIRE(ldql >= rows && ldx >= rows && ldqr >= cols, "leading dimensions are too small");
  void* ws = nullptr;
  int rc = resolve_workspace(workspace, workspace_bytes, soapmi_rotate_workspace_bytes(rows, cols), &ws);
  if (rc) return rc;
  Workspace w(ws, soapmi_rotate_workspace_bytes(rows, cols));
  float* h = w.take<float>((size_t)rows * cols);
  hipStream_t s = (hipStream_t)stream;
  const int m = (int)rows, n = (int)cols;
  // forward : H = QL^T X ; X = H QR        backward : H = QL X ; X = H QR^T
  rc = gemm<float>(s, forward ? 1 : 0, 0, m, n, m, 1.0f, ql, ldql, x, ldx, 0.0f, h, rows);
  if (rc) return rc;
  return gemm<float>(s, 0, forward ? 0 : 1, m, n, n, 1.0f, h, rows, qr, ldqr, 0.0f, x, ldx);
}

int soapmi_adam_f32(const float* gradient, int64_t ldg, float* momentum, int64_t ldm, float* variance,
                    int64_t ldv, float* update, int64_t ldu, int64_t rows, int64_t cols, int64_t step,
                    double beta1, double beta2, double eps, void* stream) {
  int rc = check_adam_args(step, beta1, beta2, eps);
  if (rc) return rc;
  SOAPMI_REQUIRE(rows >= 0 && cols >= 0, "matrix dimensions must be non-negative");
  if (rows == 0 || cols == 0) return kOk;
  SOAPMI_REQUIRE(gradient && momentum && variance && update, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(ldg >= rows && ldm >= rows && ldv >= rows && ldu >= rows, "leading dimensions are too small");
  AdamScalars sc = make_adam_scalars(step, beta1, beta2, eps);
  unsigned gy = (unsigned)(cols < 4096 ? cols : 4096);
  hipLaunchKernelGGL(adam_kernel, dim3((unsigned)ceil_div64(rows, 256), gy), dim3(256), 0, (hipStream_t)stream,
                     gradient, ldg, momentum, ldm, variance, ldv, update, ldu, (int)rows, (int)cols, sc);
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

size_t soapmi_rotate_adam_rotate_workspace_bytes(int64_t rows, int64_t cols) {
  WorkspaceSizer w;
  w.take<float>((size_t)rows * cols);
  w.take<float>((size_t)rows * cols);
  return w.total();
}

// The four chained products of soapmi_rotate_adam_rotate_f32 on two caller- or library-provided
// rows x cols temporaries.
static int rotate_adam_rotate_chain(const float* gradient, int64_t ldg, float* update, int64_t ldu, const float* ql,
                                    int64_t ldql, const float* qr, int64_t ldqr, float* momentum, int64_t ldm,
                                    float* variance, int64_t ldv, int64_t rows, int64_t cols, int64_t step,
                                    double beta1, double beta2, double eps, float* h, float* u, hipStream_t s) {
  const int m = (int)rows, n = (int)cols;
  const double bc2 = 1.0 - pow(beta2, (double)step);
  AdamScalars sc = make_adam_scalars(step, beta1, beta2, eps / sqrt(bc2));

  // 1. H = QL^T G.  The row-major gradient is the column-major matrix S = G^T (cols x rows, ld ldg),
  //    so op(B) = S^T.
  int rc = gemm<float>(s, 1, 1, m, n, m, 1.0f, ql, ldql, gradient, ldg, 0.0f, h, rows);
  if (rc) return rc;
  // 2. U = adam(H QR): the rotated gradient stays in the accumulators.
  {
    EpiAdam epi{momentum, variance, u, ldm, ldv, rows, sc};
    if (prefer_small_tile<float>(m, n, false)) {
      using Small = SmallTile<float>::type;
      GemmProblem<float> prob = make_problem<float, Small>(0, 0, m, n, n, h, rows, qr, ldqr, false);
      rc = launch_gemm<float, EpiAdam, Small>(s, prob, epi, 1);
    } else {
      GemmProblem<float> prob = make_problem<float>(0, 0, m, n, n, h, rows, qr, ldqr, false);
      rc = launch_gemm<float>(s, prob, epi, 1);
    }
    if (rc) return rc;
  }
  // 3. H = QL U
  rc = gemm<float>(s, 0, 0, m, n, m, 1.0f, ql, ldql, u, rows, 0.0f, h, rows);
  if (rc) return rc;
  // 4. update (row-major) = H QR^T, i.e. the column-major cols x rows matrix QR H^T.
  return gemm<float>(s, 0, 1, n, m, n, 1.0f, qr, ldqr, h, rows, 0.0f, update, ldu);
}

static int check_rotate_adam_rotate_args(const float* gradient, int64_t ldg, float* update, int64_t ldu,
                                         const float* ql, int64_t ldql, const float* qr, int64_t ldqr,
                                         float* momentum, int64_t ldm, float* variance, int64_t ldv, int64_t rows,
                                         int64_t cols, int64_t step, double beta1, double beta2, double eps) {
  int rc = check_adam_args(step, beta1, beta2, eps);
  if (rc) return rc;
  SOAPMI_REQUIRE(gradient && update && ql && qr && momentum && variance, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(rows > 0 && cols > 0, "matrix dimensions must be positive");
  SOAPMI_REQUIRE(ldg >= cols && ldu >= cols, "row-major leading dimensions are too small");
  SOAPMI_REQUIRE(ldql >= rows && ldqr >= cols && ldm >= rows && ldv >= rows, "leading dimensions are too small");
  return kOk;
}

int soapmi_rotate_adam_rotate_f32(const float* gradient, int64_t ldg, float* update, int64_t ldu, const float* ql,
                                  int64_t ldql, const float* qr, int64_t ldqr, float* momentum, int64_t ldm,
                                  float* variance, int64_t ldv, int64_t rows, int64_t cols, int64_t step,
                                  double beta1, double beta2, double eps, void* workspace,
                                  size_t workspace_bytes, void* stream) {
  int rc = check_rotate_adam_rotate_args(gradient, ldg, update, ldu, ql, ldql, qr, ldqr, momentum, ldm, variance,
                                         ldv, rows, cols, step, beta1, beta2, eps);
  if (rc) return rc;
  const size_t need = soapmi_rotate_adam_rotate_workspace_bytes(rows, cols);
  void* ws = nullptr;
  rc = resolve_workspace(workspace, workspace_bytes, need, &ws);
  if (rc) return rc;
  Workspace w(ws, need);
  float* h = w.take<float>((size_t)rows * cols);
  float* u = w.take<float>((size_t)rows * cols);
  return rotate_adam_rotate_chain(gradient, ldg, update, ldu, ql, ldql, qr, ldqr, momentum, ldm, variance, ldv, rows,
                                  cols, step, beta1, beta2, eps, h, u, (hipStream_t)stream);
}

int soapmi_rotate_adam_rotate_static_f32(const float* gradient, int64_t ldg, float* update, int64_t ldu,
                                         const float* ql, int64_t ldql, const float* qr, int64_t ldqr,
                                         float* momentum, int64_t ldm, float* variance, int64_t ldv, int64_t rows,
                                         int64_t cols, int64_t step, double beta1, double beta2, double eps,
                                         void* stream) {
  int rc = check_rotate_adam_rotate_args(gradient, ldg, update, ldu, ql, ldql, qr, ldqr, momentum, ldm, variance,
                                         ldv, rows, cols, step, beta1, beta2, eps);
  if (rc) return rc;
  SOAPMI_REQUIRE(rows * cols <= kStaticScratchElements,
                 "rows * cols = %lld exceeds the %lld elements the static scratch holds; use "
                 "soapmi_rotate_adam_rotate_f32 with a caller workspace",
                 (long long)(rows * cols), (long long)kStaticScratchElements);
  float* base = nullptr;
  rc = static_scratch_address(&base);
  if (rc) return rc;
  // Both temporaries are written in full (beta = 0 products) before anything reads them, so the
  // previous call's contents need no clearing.
  float* h = base;
  float* u = base + kStaticScratchElements;
  return rotate_adam_rotate_chain(gradient, ldg, update, ldu, ql, ldql, qr, ldqr, momentum, ldm, variance, ldv, rows,
                                  cols, step, beta1, beta2, eps, h, u, (hipStream_t)stream);
}

int soapmi_row_major_to_col_major_f32(const float* in, int64_t ldi, float* out, int64_t ldo, int64_t rows,
                                      int64_t cols, void* stream) {
  SOAPMI_REQUIRE(rows >= 0 && cols >= 0, "matrix dimensions must be non-negative");
  if (rows == 0 || cols == 0) return kOk;
  SOAPMI_REQUIRE(in && out, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(ldi >= cols && ldo >= rows, "leading dimensions are too small");
  // `in` is the column-major cols x rows matrix S; out = S^T.
  hipLaunchKernelGGL((transpose_kernel<float>), dim3((unsigned)ceil_div64(cols, 64), (unsigned)ceil_div64(rows, 64)),
                     dim3(256), 0, (hipStream_t)stream, in, ldi, out, ldo, (int)cols, (int)rows,
                     transpose_vec_ok<float>(in, ldi, out, ldo, cols, rows));
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

int soapmi_col_major_to_row_major_f32(const float* in, int64_t ldi, float* out, int64_t ldo, int64_t rows,
                                      int64_t cols, void* stream) {
  SOAPMI_REQUIRE(rows >= 0 && cols >= 0, "matrix dimensions must be non-negative");
  if (rows == 0 || cols == 0) return kOk;
  SOAPMI_REQUIRE(in && out, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(ldi >= rows && ldo >= cols, "leading dimensions are too small");
  hipLaunchKernelGGL((transpose_kernel<float>), dim3((unsigned)ceil_div64(rows, 64), (unsigned)ceil_div64(cols, 64)),
                     dim3(256), 0, (hipStream_t)stream, in, ldi, out, ldo, (int)rows, (int)cols,
                     transpose_vec_ok<float>(in, ldi, out, ldo, rows, cols));
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}


// ---- basis refresh ---------------------------------------------------------------------------

int soapmi_symm_f32(const float* a, const float* q, float* work, int64_t n, int64_t lda, int64_t ldq, int64_t ldw,
                    void* stream) {
  SOAPMI_REQUIRE(a && q && work, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(n > 0 && lda >= n && ldq >= n && ldw >= n, "matrix size and leading dimensions must be positive");
  return gemm<float>((hipStream_t)stream, 0, 0, (int)n, (int)n, (int)n, 1.0f, a, lda, q, ldq, 0.0f, work, ldw);
}

int soapmi_column_dots_f32(const float* q, int64_t ldq, const float* work, int64_t ldw, int64_t rows, int64_t cols,
                           float* estimates, void* stream) {
  SOAPMI_REQUIRE(rows >= 0 && cols >= 0, "matrix dimensions must be non-negative");
  if (cols == 0) return kOk;
  SOAPMI_REQUIRE(q && work && estimates, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(ldq >= rows && ldw >= rows, "leading dimensions are too small");
  const int vectors = aligned16_columns(q, ldq, rows) && aligned16_columns(work, ldw, rows) ? 1 : 0;
  hipLaunchKernelGGL((coldot_kernel<float>), dim3((unsigned)ceil_div64(cols, 4)), dim3(256), 0, (hipStream_t)stream, q, ldq,
                     work, ldw, (int)rows, (int)cols, estimates, vectors);
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

static int next_pow2(int64_t n) {
  int p = 1;
  while (p < n) p <<= 1;
  return p;
}

size_t soapmi_argsort_workspace_bytes(int64_t n) {
  const int np2 = next_pow2(n);
  WorkspaceSizer w;
  if (n > kArgsortRankMax) {  // the global-memory bitonic network
    w.take<float>((size_t)np2);
    w.take<int>((size_t)np2);
  }
  return w.total();
}

int soapmi_argsort_desc_f32(const float* keys, int64_t n, int64_t* order, void* workspace, size_t workspace_bytes,
                            void* stream) {
  SOAPMI_REQUIRE(n >= 0 && n < (1 << 30), "key count out of range");
  if (n == 0) return kOk;
  SOAPMI_REQUIRE(keys && order, "buffer addresses must be nonzero");
  hipStream_t s = (hipStream_t)stream;
  const int np2 = next_pow2(n);
  if (n <= kArgsortRankMax) {
    const size_t lds = (size_t)((n + 3) & ~(int64_t)3) * sizeof(unsigned);  // all keys, at most 64 KB
    hipLaunchKernelGGL(argsort_desc_rank_kernel, dim3((unsigned)ceil_div64(n, 64)), dim3(256), lds, s, keys, (int)n, order);
    SOAPMI_LAUNCH_CHECK();
    return kOk;
  }
  const size_t need = soapmi_argsort_workspace_bytes(n);
  void* ws = nullptr;
  int rc = resolve_workspace(workspace, workspace_bytes, need, &ws);
  if (rc) return rc;
  Workspace w(ws, need);
  float* v = w.take<float>((size_t)np2);
  int* id = w.take<int>((size_t)np2);
  const unsigned blocks = (unsigned)ceil_div64(np2, 256);
  hipLaunchKernelGGL(argsort_init_kernel, dim3(blocks), dim3(256), 0, s, keys, (int)n, np2, v, id);
  for (int k = 2; k <= np2; k <<= 1)
    for (int j = k >> 1; j > 0; j >>= 1)
      hipLaunchKernelGGL(argsort_stage_kernel, dim3(blocks), dim3(256), 0, s, v, id, np2, k, j);
  hipLaunchKernelGGL(argsort_finish_kernel, dim3((unsigned)ceil_div64(n, 256)), dim3(256), 0, s, id, (int)n, order);
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

int soapmi_gather_f32(const float* in, int64_t ldi, float* out, int64_t ldo, int64_t rows, int64_t cols,
                      const int64_t* row_order, const int64_t* col_order, void* stream) {
  SOAPMI_REQUIRE(rows >= 0 && cols >= 0, "matrix dimensions must be non-negative");
  if (rows == 0 || cols == 0) return kOk;
  SOAPMI_REQUIRE(in && out && in != out, "buffers must be nonzero and distinct");
  SOAPMI_REQUIRE(ldi >= rows && ldo >= rows, "leading dimensions are too small");
  launch_gather2d((hipStream_t)stream, in, ldi, out, ldo, rows, cols, row_order, col_order);
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

size_t soapmi_permute_workspace_bytes(int64_t rows, int64_t cols) {
  WorkspaceSizer w;
  w.take<float>((size_t)rows * cols);
  return w.total();
}

static int permute_with(hipStream_t s, float* matrix, int64_t ld, int64_t rows, int64_t cols,
                        const int64_t* row_order, const int64_t* col_order, float* tmp) {
  launch_gather2d(s, matrix, ld, tmp, rows, rows, cols, row_order, col_order);
  launch_gather2d(s, tmp, rows, matrix, ld, rows, cols, nullptr, nullptr);  // copy back
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

int soapmi_permute_f32(float* matrix, int64_t ld, int64_t rows, int64_t cols, const int64_t* row_order,
                       const int64_t* col_order, void* workspace, size_t workspace_bytes, void* stream) {
  SOAPMI_REQUIRE(rows >= 0 && cols >= 0, "matrix dimensions must be non-negative");
  if (rows == 0 || cols == 0) return kOk;
  SOAPMI_REQUIRE(matrix, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(ld >= rows, "leading dimension is too small");
  const size_t need = soapmi_permute_workspace_bytes(rows, cols);
  void* ws = nullptr;
  int rc = resolve_workspace(workspace, workspace_bytes, need, &ws);
  if (rc) return rc;
  Workspace w(ws, need);
  float* tmp = w.take<float>((size_t)rows * cols);
  return permute_with((hipStream_t)stream, matrix, ld, rows, cols, row_order, col_order, tmp);
}

int soapmi_is_permutation(const int64_t* order, int64_t n, void* workspace, size_t workspace_bytes, void* stream) {
  SOAPMI_REQUIRE(n >= 0 && n < (1ll << 31), "size out of range");
  if (n == 0) return 1;
  SOAPMI_REQUIRE(order, "buffer addresses must be nonzero");
  const size_t need = (size_t)(n + 1) * sizeof(int) + 512;
  void* ws = nullptr;
  int rc = resolve_workspace(workspace, workspace_bytes, need, &ws);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  int* seen = static_cast<int*>(ws);
  int* flag = seen + n;
  SOAPMI_HIP(hipMemsetAsync(seen, 0, (size_t)(n + 1) * sizeof(int), s));
  hipLaunchKernelGGL(check_permutation_kernel, dim3((unsigned)ceil_div64(n, 256)), dim3(256), 0, s, order, (int)n, seen,
                     flag);
  SOAPMI_LAUNCH_CHECK();
  int host_flag = 0;
  SOAPMI_HIP(hipMemcpyAsync(&host_flag, flag, sizeof(int), hipMemcpyDeviceToHost, s));
  SOAPMI_HIP(hipStreamSynchronize(s));
  return host_flag ? 0 : 1;
}

size_t soapmi_qr_workspace_bytes(int64_t n) { return qr_workspace_bytes<float>(n); }

int soapmi_qr_f32(float* matrix, float* q, int64_t n, int64_t ldmatrix, int64_t ldq, void* workspace,
                  size_t workspace_bytes, void* stream) {
  SOAPMI_REQUIRE(matrix && q, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(n > 0 && ldmatrix > 0 && ldq > 0, "matrix size and leading dimensions must be positive");
  SOAPMI_REQUIRE(ldmatrix >= n && ldq >= n, "leading dimensions are too small");
  SOAPMI_REQUIRE(matrix != q, "matrix and q must not overlap");
  const size_t need = soapmi_qr_workspace_bytes(n);
  void* ws = nullptr;
  int rc = resolve_workspace(workspace, workspace_bytes, need, &ws);
  if (rc) return rc;
  Workspace w(ws, need);
  QrWorkspace<float> qws;
  qr_workspace_layout<float>(w, n, &qws);
  int* report = nullptr;
  rc = failure_report(&report);
  if (rc) return rc;
  PersistentGuard guard;
  rc = guard.acquire((hipStream_t)stream, (int)ceil_div64(n, 256));
  if (rc) return rc;
  rc = qr_factor_and_form_q<float>((hipStream_t)stream, matrix, ldmatrix, q, ldq, (int)n, qws,
                                   std::min(g_qr_persistent_max_wg.load(), compute_unit_count()),
                                   g_message_spin_limit.load(),
                                   g_qr_columns_per_round.load(), report, g_qr_carry_update.load() != 0,
                                   g_qr_super_block.load());
  const int rc_release = guard.release();
  return rc ? rc : rc_release;
}

size_t soapmi_power_iteration_qr_workspace_bytes(int64_t n) {
  WorkspaceSizer w;
  w.take<float>((size_t)n * n);  // gather target
  w.take<float>((size_t)n);      // estimates
  w.take<char>(soapmi_argsort_workspace_bytes(n));
  w.take<char>(soapmi_qr_workspace_bytes(n));
  return w.total();
}

int soapmi_power_iteration_qr_f32(float* p, float* q, float* work, int64_t n, int64_t ldp, int64_t ldq,
                                  int64_t ldw, int symmetrize, int64_t* order, float* estimates, void* workspace,
                                  size_t workspace_bytes, void* stream) {
  SOAPMI_REQUIRE(p && q && work && order, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(n > 0 && ldp >= n && ldq >= n && ldw >= n, "matrix size and leading dimensions must be positive");
  SOAPMI_REQUIRE(p != q && p != work && q != work, "preconditioner, Q, and work must not overlap.");
  const size_t need = soapmi_power_iteration_qr_workspace_bytes(n);
  void* ws = nullptr;
  int rc = resolve_workspace(workspace, workspace_bytes, need, &ws);
  if (rc) return rc;
  Workspace w(ws, need);
  float* tmp = w.take<float>((size_t)n * n);
  float* est = w.take<float>((size_t)n);
  const size_t sort_bytes = soapmi_argsort_workspace_bytes(n);
  char* sort_ws = w.take<char>(sort_bytes);
  const size_t qr_bytes = soapmi_qr_workspace_bytes(n);
  char* qr_ws = w.take<char>(qr_bytes);
  hipStream_t s = (hipStream_t)stream;
  if (symmetrize) {
    rc = soapmi_symmetrize_lower_f32(p, n, ldp, stream);
    if (rc) return rc;
  }
  rc = soapmi_symm_f32(p, q, work, n, ldp, ldq, ldw, stream);
  if (rc) return rc;
  rc = soapmi_column_dots_f32(q, ldq, work, ldw, n, n, est, stream);
  if (rc) return rc;
  if (estimates) SOAPMI_HIP(hipMemcpyAsync(estimates, est, (size_t)n * sizeof(float), hipMemcpyDeviceToDevice, s));
  rc = soapmi_argsort_desc_f32(est, n, order, sort_ws, sort_bytes, stream);
  if (rc) return rc;
  rc = permute_with(s, work, ldw, n, n, nullptr, order, tmp);
  if (rc) return rc;
  return soapmi_qr_f32(work, q, n, ldw, ldq, qr_ws, qr_bytes, stream);
}

size_t soapmi_refresh_workspace_bytes(int64_t rows, int64_t cols) {
  // the two factorisation chains run concurrently and need disjoint scratch; the rotations and
  // the variance permutation before and after them reuse the same bytes
  WorkspaceSizer chains;
  chains.take<char>(soapmi_power_iteration_qr_workspace_bytes(rows));
  chains.take<char>(soapmi_power_iteration_qr_workspace_bytes(cols));
  size_t m = chains.total();
  const size_t a = soapmi_rotate_workspace_bytes(rows, cols);
  const size_t d = soapmi_permute_workspace_bytes(rows, cols);
  m = m > a ? m : a;
  return m > d ? m : d;
}

int soapmi_refresh_f32(float* momentum, int64_t ldm, float* variance, int64_t ldv, float* left_preconditioner,
                       int64_t ldl, float* right_preconditioner, int64_t ldr, float* q_left, int64_t ldql,
                       float* q_right, int64_t ldqr, float* left_work, int64_t ldlw, float* right_work,
                       int64_t ldrw, int64_t rows, int64_t cols, int symmetrize, int64_t* left_order,
                       int64_t* right_order, void* workspace, size_t workspace_bytes, void* stream) {
  SOAPMI_REQUIRE(momentum && variance && left_order && right_order, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(rows > 0 && cols > 0, "matrix dimensions must be positive");
  const size_t need = soapmi_refresh_workspace_bytes(rows, cols);
  void* ws = nullptr;
  int rc = resolve_workspace(workspace, workspace_bytes, need, &ws);
  if (rc) return rc;
  SideStream* side = nullptr;
  rc = side_stream(&side);
  if (rc) return rc;
  hipStream_t main_stream = (hipStream_t)stream;
  Workspace chains(ws, need);
  const size_t left_bytes = soapmi_power_iteration_qr_workspace_bytes(rows);
  const size_t right_bytes = soapmi_power_iteration_qr_workspace_bytes(cols);
  char* left_ws = chains.take<char>(left_bytes);
  char* right_ws = chains.take<char>(right_bytes);

  rc = soapmi_rotate_f32(q_left, momentum, q_right, rows, cols, ldql, ldm, ldqr, 0, ws, need, stream);
  if (rc) return rc;
  // fork: the smaller chain goes to the side stream, whose latency-bound panel kernels fill the
  // gaps of the larger one
  const bool two_streams = g_refresh_streams.load() == 2;
  const bool left_on_side = rows <= cols;
  void* const side_or_main = two_streams ? (void*)side->stream : stream;
  if (two_streams) {
    SOAPMI_HIP(hipEventRecord(side->fork, main_stream));
    SOAPMI_HIP(hipStreamWaitEvent(side->stream, side->fork, 0));
  }
  int rc_left = soapmi_power_iteration_qr_f32(left_preconditioner, q_left, left_work, rows, ldl, ldql, ldlw, symmetrize,
                                              left_order, nullptr, left_ws, left_bytes,
                                              left_on_side ? side_or_main : stream);
  int rc_right = kOk;
  if (rc_left == kOk)
    rc_right = soapmi_power_iteration_qr_f32(right_preconditioner, q_right, right_work, cols, ldr, ldqr, ldrw,
                                             symmetrize, right_order, nullptr, right_ws, right_bytes,
                                             left_on_side ? stream : side_or_main);
  // join, also after a failure: nothing may stay detached from the caller's stream
  if (two_streams) {
    SOAPMI_HIP(hipEventRecord(side->join, side->stream));
    SOAPMI_HIP(hipStreamWaitEvent(main_stream, side->join, 0));
  }
  if (rc_left) return rc_left;
  if (rc_right) return rc_right;
  rc = soapmi_permute_f32(variance, ldv, rows, cols, left_order, right_order, ws, need, stream);
  if (rc) return rc;
  return soapmi_rotate_f32(q_left, momentum, q_right, rows, cols, ldql, ldm, ldqr, 1, ws, need, stream);
}


// ---- eigensolver ------------------------------------------------------------------------------

size_t soapmi_eigh_workspace_bytes(int64_t n, int element_bytes) {
  return element_bytes == 8 ? eigh_workspace_bytes_any<double>(n) : eigh_workspace_bytes_any<float>(n);
}

int soapmi_eigh_f64(double* a, double* eigenvalues, double* q, int64_t n, int64_t lda, int64_t ldq,
                    void* workspace, size_t workspace_bytes, void* stream) {
  return eigh_entry<double>(a, eigenvalues, q, n, lda, ldq, workspace, workspace_bytes, stream);
}

int soapmi_eigh_f32(float* a, float* eigenvalues, float* q, int64_t n, int64_t lda, int64_t ldq, void* workspace,
                    size_t workspace_bytes, void* stream) {
  return eigh_entry<float>(a, eigenvalues, q, n, lda, ldq, workspace, workspace_bytes, stream);
}

size_t soapmi_initialize_basis_workspace_bytes(int64_t n, int implementation) {
  WorkspaceSizer w;
  if (implementation == 0) {
    w.take<double>((size_t)n * n);
    w.take<double>((size_t)n * n);
    w.take<double>((size_t)n);
    w.take<char>(eigh_workspace_bytes_any<double>(n));
  } else {
    w.take<float>((size_t)n * n);
    w.take<float>((size_t)n * n);
    w.take<float>((size_t)n);
    w.take<char>(eigh_workspace_bytes_any<float>(n));
  }
  return w.total();
}

int soapmi_initialize_basis_f32(const float* p, float* q, float* work, float* eigenvalues, int64_t n, int64_t ldp,
                                int64_t ldq, int64_t ldw, int implementation, void* workspace,
                                size_t workspace_bytes, void* stream) {
  SOAPMI_REQUIRE(implementation == 0 || implementation == 1, "implementation must be 0 (elpa) or 1 (eigh), got %d.",
                 implementation);
  SOAPMI_REQUIRE(p && q && work && eigenvalues, "buffer addresses must be nonzero");
  SOAPMI_REQUIRE(n > 0, "matrix dimensions and block size must be positive");
  SOAPMI_REQUIRE(ldp >= n && ldq >= n && ldw >= n, "leading dimensions are too small");
  SOAPMI_REQUIRE(p != q && p != work && q != work, "preconditioner, Q, and work must not overlap.");
  const size_t need = soapmi_initialize_basis_workspace_bytes(n, implementation);
  void* ws = nullptr;
  int rc = resolve_workspace(workspace, workspace_bytes, need, &ws);
  if (rc) return rc;
  Workspace w(ws, need);
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)ceil_div64(n, 256), (unsigned)(n < 4096 ? n : 4096));
  const dim3 tiles((unsigned)ceil_div64(n, 64), (unsigned)ceil_div64(n, 64));
  const unsigned vblocks = (unsigned)ceil_div64(n, 256);
  if (implementation == 0) {
    double* a64 = w.take<double>((size_t)n * n);
    double* z64 = w.take<double>((size_t)n * n);
    double* w64 = w.take<double>((size_t)n);
    const size_t eb = eigh_workspace_bytes_any<double>(n);
    char* ebuf = w.take<char>(eb);
    // work <- -P (both triangles), then its float64 copy, as factorizations.py:500-507 stages them
    hipLaunchKernelGGL((sym_convert_kernel<float, float>), tiles, dim3(256), 0, s, p, ldp, work, ldw, (int)n, -1.0f, 0.0f);
    hipLaunchKernelGGL((sym_convert_kernel<float, double>), tiles, dim3(256), 0, s, p, ldp, a64, n, (int)n, -1.0, 0.0);
    SOAPMI_LAUNCH_CHECK();
    rc = soapmi_eigh_f64(a64, w64, z64, n, n, n, ebuf, eb, stream);
    if (rc) return rc;
    hipLaunchKernelGGL((convert_columns_kernel<double, float>), grid, dim3(256), 0, s, z64, n, q, ldq, (int)n, 0);
    hipLaunchKernelGGL((convert_vector_kernel<double, float>), dim3(vblocks), dim3(256), 0, s, w64, eigenvalues, (int)n,
                       -1.0f, 0);
  } else {
    float* a32 = w.take<float>((size_t)n * n);
    float* z32 = w.take<float>((size_t)n * n);
    float* w32 = w.take<float>((size_t)n);
    const size_t eb = eigh_workspace_bytes_any<float>(n);
    char* ebuf = w.take<char>(eb);
    hipLaunchKernelGGL((sym_convert_kernel<float, float>), tiles, dim3(256), 0, s, p, ldp, a32, n, (int)n, 1.0f, 1e-30f);
    SOAPMI_LAUNCH_CHECK();
    rc = soapmi_eigh_f32(a32, w32, z32, n, n, n, ebuf, eb, stream);
    if (rc) return rc;
    hipLaunchKernelGGL((convert_columns_kernel<float, float>), grid, dim3(256), 0, s, z32, n, q, ldq, (int)n, 1);
    hipLaunchKernelGGL((convert_vector_kernel<float, float>), dim3(vblocks), dim3(256), 0, s, w32, eigenvalues, (int)n,
                       1.0f, 1);
  }
  SOAPMI_LAUNCH_CHECK();
  return kOk;
}

}  // extern "C"
