// C ABI of libsbhip.so (see include/sbhip.h): library context, per-kernel entry points and the
// device-resident network object.  Host code only; kernels live in sb_kernels.hpp.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <utility>
#include <mutex>
#include <new>
#include <random>
#include <atomic>
#include <condition_variable>
#include <string>
#include <system_error>
#include <thread>
#include <vector>

#include "../../include/sbhip.h"
#include "sb_launch.hpp"

namespace sb {

static thread_local std::string g_error;
void set_error(const std::string &msg) { g_error = msg; }
int hip_fail(hipError_t e, const char *what, const char *file, int line) {
  g_error = std::string("HIP error '") + hipGetErrorString(e) + "' from " + what + " at " + file + ":" +
            std::to_string(line);
  return SB_ERR_HIP;
}

// Every allocating runtime call of the library goes through these, so that a caller (and the test of the
// entry point that promises to allocate nothing) can ask how many there have been: sb_allocation_calls.
static long g_allocation_calls = 0;
template <typename P>
static hipError_t dev_malloc(P **p, size_t bytes) {
  g_allocation_calls++;
  return hipMalloc((void **)p, bytes);
}
static hipError_t event_create(hipEvent_t *e) {
  g_allocation_calls++;
  return hipEventCreate(e);
}

struct Context {
  bool ready = false;
  int device = 0;
  hipStream_t stream = nullptr;
  // scratch of the per-kernel sb_update_mask entry point
  void *mask_nom = nullptr;
  int *mask_csum = nullptr;
  long mask_cap = 0;
  // scratch of the per-kernel training entry points: the "next" Ci / Cj of the fused kernel
  void *trace_next = nullptr;
  long trace_cap = 0;  // elements of 8 bytes
  // device address of `scratch` on this context's device
  void *noalloc_scratch = nullptr;
};
static Context g_ctx;
static std::mutex g_ctx_mutex;

// Host -> device copies of caller memory (pageable, as numpy arrays are) through a ring of pinned chunks: the
// bytes are copied into a pinned chunk by several host threads at once, and the chunk goes to the device with an
// asynchronous copy while the threads fill the next one.  (One synchronous copy straight from pageable memory
// runs at about 21 GB/s here; the reference's loader keeps pinned double buffers for the same reason,
// full_cuda_backend/dataloader.h:36-212.)  The pinned chunks are allocated on first use and kept until
// sb_shutdown.
// The host threads that fill a pinned chunk: kThreads - 1 workers that sleep between jobs, plus the caller.
// The pool lives on the heap and its threads are detached: a process that ends without sb_shutdown must not
// find joinable threads in a static object.  On release the workers are told to leave; the few bytes of the
// pool itself stay allocated, so that a worker that wakes late still finds its flags.
struct CopyPool {
  static constexpr int kThreads = 8;
  std::mutex m;
  std::condition_variable go, done;
  unsigned long generation = 0;
  int pending = 0;
  bool stop = false;
  char *dst = nullptr;
  const char *src = nullptr;
  size_t bytes = 0, piece = 0;
  void worker(int index) {
    unsigned long seen = 0;
    for (;;) {
      std::unique_lock<std::mutex> lock(m);
      go.wait(lock, [&] { return stop || generation != seen; });
      if (stop) return;
      seen = generation;
      const size_t at = (size_t)index * piece;
      char *d = dst;
      const char *sp = src;
      const size_t n = at < bytes ? std::min(piece, bytes - at) : 0;
      lock.unlock();
      if (n) std::memcpy(d + at, sp + at, n);
      lock.lock();
      if (--pending == 0) done.notify_one();
    }
  }
  int workers = 0;  // started; a thread the system refuses is done without
  void start() {
    for (int k = 1; k < kThreads; k++) {
      try {
        std::thread([this, k] { worker(k); }).detach();
      } catch (const std::system_error &) {
        break;
      }
      workers = k;
    }
  }
  // copies bytes in pieces of whole pages, one per thread; returns when all of them are done
  void copy(void *d, const void *sp, size_t n) {
    if (n < ((size_t)1 << 20) || workers == 0) {
      std::memcpy(d, sp, n);
      return;
    }
    {
      std::lock_guard<std::mutex> lock(m);
      dst = (char *)d;
      src = (const char *)sp;
      bytes = n;
      piece = ((n / (size_t)(workers + 1)) + 4095) & ~(size_t)4095;
      pending = workers;
      generation++;
    }
    go.notify_all();
    std::memcpy(d, sp, std::min(piece, n));  // the caller's piece
    std::unique_lock<std::mutex> lock(m);
    done.wait(lock, [&] { return pending == 0; });
  }
  void leave() {
    {
      std::lock_guard<std::mutex> lock(m);
      stop = true;
    }
    go.notify_all();
  }
};

struct HostStager {
  static constexpr int kChunks = 4;
  static constexpr size_t kChunkBytes = (size_t)8 << 20;
  void *pinned[kChunks] = {nullptr, nullptr, nullptr, nullptr};
  hipEvent_t sent[kChunks] = {nullptr, nullptr, nullptr, nullptr};  // the chunk's copy to the device has finished
  CopyPool *pool = nullptr;
  hipStream_t copy_stream = nullptr;  // for uploads that run beside the library stream's kernels
  hipEvent_t uploaded = nullptr, consumed = nullptr;
  int next = 0;
  bool ready = false;
};
static HostStager g_stager;

static int stager_init() {
  if (g_stager.ready) return 0;
  for (int k = 0; k < HostStager::kChunks; k++) {
    g_allocation_calls += 2;
    SB_HIP(hipHostMalloc(&g_stager.pinned[k], HostStager::kChunkBytes, hipHostMallocDefault));
    SB_HIP(hipEventCreateWithFlags(&g_stager.sent[k], hipEventDisableTiming));
  }
  g_allocation_calls += 3;
  SB_HIP(hipStreamCreate(&g_stager.copy_stream));  // (default priority, like the library's stream)
  SB_HIP(hipEventCreateWithFlags(&g_stager.uploaded, hipEventDisableTiming));
  SB_HIP(hipEventCreateWithFlags(&g_stager.consumed, hipEventDisableTiming));
  g_stager.pool = new CopyPool();
  g_stager.pool->start();
  g_stager.ready = true;
  return 0;
}

static void stager_release() {
  for (int k = 0; k < HostStager::kChunks; k++) {
    if (g_stager.pinned[k]) (void)hipHostFree(g_stager.pinned[k]);
    if (g_stager.sent[k]) (void)hipEventDestroy(g_stager.sent[k]);
    g_stager.pinned[k] = nullptr;
    g_stager.sent[k] = nullptr;
  }
  if (g_stager.copy_stream) (void)hipStreamDestroy(g_stager.copy_stream);
  if (g_stager.uploaded) (void)hipEventDestroy(g_stager.uploaded);
  if (g_stager.consumed) (void)hipEventDestroy(g_stager.consumed);
  if (g_stager.pool) g_stager.pool->leave();  // (not deleted: see CopyPool)
  g_stager = HostStager();
}

// d_dst[0 .. bytes) = h_src[0 .. bytes), ordered on stream `st`.  Returns once h_src has been read (the caller
// may reuse it); the last chunks may still be on their way to the device, in stream order.
static int staged_upload(void *d_dst, const void *h_src, size_t bytes, hipStream_t st) {
  if (bytes == 0) return 0;
  int rc = stager_init();
  if (rc) return rc;
  for (size_t at = 0; at < bytes; at += HostStager::kChunkBytes) {
    const size_t n = std::min(HostStager::kChunkBytes, bytes - at);
    const int k = g_stager.next;
    g_stager.next = (k + 1) % HostStager::kChunks;
    SB_HIP(hipEventSynchronize(g_stager.sent[k]));  // (an event never recorded counts as finished)
    g_stager.pool->copy(g_stager.pinned[k], (const char *)h_src + at, n);
    SB_HIP(hipMemcpyAsync((char *)d_dst + at, g_stager.pinned[k], n, hipMemcpyHostToDevice, st));
    SB_HIP(hipEventRecord(g_stager.sent[k], st));
  }
  return 0;
}

// Scratch of sb_update_weights_noalloc_f32: the "next" Ci / Cj of the fused kernel for callers that
// cannot allocate.  Part of the loaded code object, so every GPU the library runs on holds its own copy
// until the process ends.  In host code the array's name is only a handle: sb_init asks the runtime for
// the device address once (g_ctx.noalloc_scratch) and everything below uses that.
static __device__ __align__(256) unsigned char scratch[SB_NOALLOC_MAX_UNITS * sizeof(float)];

// ---- per-kernel event timing (sb_profile_start / sb_profile_stop)
struct ProfRecord {
  int id;
  hipEvent_t start, stop;
};
static bool g_prof_on = false;
static std::vector<ProfRecord> g_prof_records;
static std::vector<hipEvent_t> g_prof_pool;
static double g_prof_ms[K_COUNT];
static long g_prof_launches[K_COUNT];
static double g_prof_overhead_ms = 0;  // elapsed time of an empty event bracket

const char *kernel_name(int id) {
  static const char *names[K_COUNT] = {"forward", "softmax", "update_bias",
                                       "update_bias_regularized", "mask_scores", "mask_swap",
                                       "mask_fix_weights", "apply_mask", "argmax", "gather_rows", "fill",
                                       "train_fused", "mask_rows", "weight_pass"};
  return (id >= 0 && id < K_COUNT) ? names[id] : "?";
}

static hipEvent_t prof_event() {
  hipEvent_t e = nullptr;
  if (!g_prof_pool.empty()) {
    e = g_prof_pool.back();
    g_prof_pool.pop_back();
  } else if (event_create(&e) != hipSuccess) {
    e = nullptr;
  }
  return e;
}

// Under rocprofv3 (which sets ROCPROF_OUTPUT_PATH for the program it runs) the dispatch timestamps belong to the
// profiler and events carried by a launch read long (29 us for a 16 us kernel): the scopes bracket then.
static bool g_prof_carry = true;
ProfScope::ProfScope(hipStream_t st, int id, bool carried)
    : st_(st), slot_(-1), carried_(carried && g_prof_carry) {
  carried = carried_;
  if (!g_prof_on) return;
  ProfRecord r{id, prof_event(), prof_event()};
  if (!r.start || !r.stop) return;
  if (!carried) (void)hipEventRecord(r.start, st);
  g_prof_records.push_back(r);
  slot_ = (int)g_prof_records.size() - 1;
}
ProfScope::~ProfScope() {
  if (slot_ >= 0 && !carried_) (void)hipEventRecord(g_prof_records[slot_].stop, st_);
}
hipEvent_t ProfScope::start() const { return slot_ >= 0 ? g_prof_records[slot_].start : nullptr; }
hipEvent_t ProfScope::stop() const { return slot_ >= 0 ? g_prof_records[slot_].stop : nullptr; }
bool prof_carried(int id) { return g_prof_carry && id == K_TRAIN_FUSED; }

static int require_ready() {
  if (!g_ctx.ready) {
    set_error("sb_init has not been called");
    return SB_ERR_STATE;
  }
  return 0;
}

#define SB_READY()          \
  do {                      \
    int rc_ = require_ready(); \
    if (rc_) return rc_;    \
  } while (0)

static int ensure_mask_scratch(long N) {
  if (N <= g_ctx.mask_cap) return 0;
  SB_HIP(hipStreamSynchronize(g_ctx.stream));
  if (g_ctx.mask_nom) SB_HIP(hipFree(g_ctx.mask_nom));
  if (g_ctx.mask_csum) SB_HIP(hipFree(g_ctx.mask_csum));
  g_ctx.mask_nom = nullptr;
  g_ctx.mask_csum = nullptr;
  g_ctx.mask_cap = 0;
  SB_HIP(dev_malloc(&g_ctx.mask_nom, (size_t)N * sizeof(double)));
  SB_HIP(dev_malloc((void **)&g_ctx.mask_csum, (size_t)N * sizeof(int)));
  g_ctx.mask_cap = N;
  return 0;
}

static int ensure_trace_scratch(long elems) {
  if (elems <= g_ctx.trace_cap) return 0;
  SB_HIP(hipStreamSynchronize(g_ctx.stream));
  if (g_ctx.trace_next) SB_HIP(hipFree(g_ctx.trace_next));
  g_ctx.trace_next = nullptr;
  g_ctx.trace_cap = 0;
  SB_HIP(dev_malloc(&g_ctx.trace_next, (size_t)elems * sizeof(double)));
  g_ctx.trace_cap = elems;
  return 0;
}

// Per-kernel entry points keep the reference's in-place contract: the fused kernel writes the new
// Ci / Cj into scratch, which is then copied over the caller's arrays.
// `fixed_scratch`: room for N + M elements that the caller brings (no allocation here), or nullptr to
// use the context's growable buffer.
template <typename T>
static int train_in_place(const T *x, const T *y, T *Cij, T *W, T *Ci, T *Cj, const uint8_t *wmask,
                          int bias_mode, T *bias, T *kbi, long B, long N, long H, long Mc, T taupdt,
                          T cthr, T khalf, T pmin, T taubdt, T *fixed_scratch = nullptr) {
  hipStream_t st = g_ctx.stream;
  const long M = H * Mc;
  SB_REQUIRE(N > 0 && M > 0, "sizes must be positive");
  int rc = fixed_scratch ? 0 : ensure_trace_scratch(N + M);
  if (rc) return rc;
  T *ci_next = fixed_scratch ? fixed_scratch : (T *)g_ctx.trace_next, *cj_next = ci_next + N;
  rc = launch_train_fused<T>(st, x, y, Cij, W, Ci, Cj, ci_next, cj_next, wmask, bias_mode, bias, kbi, B,
                             N, H, Mc, taupdt, cthr, khalf, pmin, taubdt, false);
  if (rc) return rc;
  return launch_copy_pair<T>(st, Ci, ci_next, (size_t)N, Cj, cj_next, (size_t)M);
}

// ======================================================================================== network
struct Layer {
  bool plastic = false;
  long N = 0, H = 0, Mc = 0, M = 0;
  double taupdt = 0, pmin = 0, khalf = 0, taubdt = 0;
  void *W = nullptr, *bias = nullptr, *Ci = nullptr, *Cj = nullptr, *Cij = nullptr, *kbi = nullptr;
  void *Ci_alt = nullptr, *Cj_alt = nullptr;  // the fused training kernel ping-pongs Ci / Cj
  uint8_t *wmask = nullptr;
  void *act = nullptr;  // [act_rows, M]
  long act_rows = 0;
  void *nom = nullptr;  // rewiring scratch [N]
  int *csum = nullptr;
  // Sparse layers (at most 70 % of wmask set): per-hypercolumn lists of the connected rows for the
  // forward pass, kept in step with wmask.  They are used while W is known to be zero wherever wmask
  // is 0, which a training step establishes and a write to W or wmask through the state interface
  // ends.
  int *rows = nullptr, *row_cnt = nullptr;
  long rows_cap = 0;
  bool w_masked = false;
  bool w_unchecked = false;  // W or wmask came from outside and has not been looked at yet
};

}  // namespace sb

struct sb_net {
  int dtype = SB_F32;
  size_t esize = 4;
  std::vector<sb::Layer> layers;
  // training set in HBM, its per-epoch permuted copy and the permutation
  void *X = nullptr, *Y = nullptr, *Xp = nullptr, *Yp = nullptr;
  long XpB_batch = 0;   // batch size XpB is valid for in the current epoch (0: not valid)
  void *XpB = nullptr;  // Xp in blocks of 16 rows (k_gather_rows_blocked), for the first layer's forward over row lists
  long Ns = 0, NF = 0, NC = 0;
  int64_t *d_perm = nullptr;
  int64_t *h_perm = nullptr;  // pinned staging
  hipEvent_t perm_copied = nullptr;
  // While only the last layer trains, the layers below it are frozen: their output for every training
  // sample is computed once (Hc, data-set order) and shuffled per epoch like the images (Hcp).
  void *Hc = nullptr, *Hcp = nullptr;
  int Hc_layer = -1;  // Hc holds the activations of this layer for the current training set (-1: none)
  size_t frozen_cache_limit = (size_t)16 << 30;  // bytes, both copies together (sb_net_set_frozen_cache_limit)
  unsigned long long *d_correct = nullptr;   // evaluate's counter
  unsigned long long *d_unmasked = nullptr;  // layer_check_masked's counter
  // evaluate / predict / forward: the device buffers of one chunk of the set (images, the same in blocks of 16
  // rows, labels, predictions), kept from call to call (an allocation and a release per buffer and call took a
  // fifth of an evaluate of 10000 images) and released with the network
  struct Reusable {
    void *p = nullptr;
    size_t cap = 0;
  } ev_x, ev_xb, ev_y, ev_p;
};

namespace sb {

static inline long cdiv_l(long a, long b) { return (a + b - 1) / b; }

// Device allocation that is released when the scope ends, whichever way it ends.
struct ScopedDeviceBuffer {
  void *p = nullptr;
  ScopedDeviceBuffer() = default;
  ScopedDeviceBuffer(const ScopedDeviceBuffer &) = delete;
  ScopedDeviceBuffer &operator=(const ScopedDeviceBuffer &) = delete;
  ~ScopedDeviceBuffer() {
    if (p) (void)hipFree(p);
  }
};

static int free_dev(void *&p) {
  if (p) SB_HIP(hipFree(p));
  p = nullptr;
  return 0;
}

// b holds at least `bytes` afterwards (contents undefined); nothing in flight may still use the old buffer
static int reuse_dev(sb_net::Reusable &b, size_t bytes) {
  if (bytes <= b.cap) return 0;
  SB_HIP(hipStreamSynchronize(g_ctx.stream));
  int rc = free_dev(b.p);
  b.cap = 0;
  if (rc) return rc;
  SB_HIP(dev_malloc(&b.p, bytes));
  b.cap = bytes;
  return 0;
}

template <typename T>
static int layer_alloc(Layer &L, T ci0, T cj0, T cij0) {
  hipStream_t st = g_ctx.stream;
  const size_t nm = (size_t)L.N * L.M;
  SB_HIP(dev_malloc(&L.W, nm * sizeof(T)));
  SB_HIP(dev_malloc(&L.Cij, nm * sizeof(T)));
  SB_HIP(dev_malloc(&L.bias, L.M * sizeof(T)));
  SB_HIP(dev_malloc(&L.Cj, L.M * sizeof(T)));
  SB_HIP(dev_malloc(&L.Ci, L.N * sizeof(T)));
  SB_HIP(dev_malloc(&L.Cj_alt, L.M * sizeof(T)));
  SB_HIP(dev_malloc(&L.Ci_alt, L.N * sizeof(T)));
  int rc = 0;
  if ((rc = launch_fill<T>(st, (T *)L.W, T(0), nm))) return rc;
  if ((rc = launch_fill<T>(st, (T *)L.Cij, cij0, nm))) return rc;
  if ((rc = launch_fill<T>(st, (T *)L.bias, T(0), L.M))) return rc;
  if ((rc = launch_fill<T>(st, (T *)L.Cj, cj0, L.M))) return rc;
  if ((rc = launch_fill<T>(st, (T *)L.Ci, ci0, L.N))) return rc;
  if (L.plastic) {
    SB_HIP(dev_malloc(&L.kbi, L.M * sizeof(T)));
    SB_HIP(dev_malloc((void **)&L.wmask, (size_t)L.N * L.H));
    SB_HIP(dev_malloc(&L.nom, L.N * sizeof(T)));
    SB_HIP(dev_malloc((void **)&L.csum, L.N * sizeof(int)));
    if ((rc = launch_fill<T>(st, (T *)L.kbi, T(1), L.M))) return rc;
    if ((rc = launch_fill_bytes(st, L.wmask, 1, (size_t)L.N * L.H))) return rc;
  }
  return 0;
}

static int layer_free(Layer &L) {
  int rc = 0;
  void *w = L.wmask, *c = L.csum;
  rc |= free_dev(L.W); rc |= free_dev(L.bias); rc |= free_dev(L.Ci); rc |= free_dev(L.Cj);
  rc |= free_dev(L.Cij); rc |= free_dev(L.kbi); rc |= free_dev(w); rc |= free_dev(L.act);
  rc |= free_dev(L.nom); rc |= free_dev(c); rc |= free_dev(L.Ci_alt); rc |= free_dev(L.Cj_alt);
  void *r = L.rows, *rc_ = L.row_cnt;
  rc |= free_dev(r); rc |= free_dev(rc_);
  L.wmask = nullptr; L.csum = nullptr; L.rows = nullptr; L.row_cnt = nullptr; L.rows_cap = 0;
  return rc;
}

static int ensure_act(sb_net *net, long rows) {
  for (auto &L : net->layers) {
    if (L.act_rows >= rows) continue;
    SB_HIP(hipStreamSynchronize(g_ctx.stream));
    int rc = free_dev(L.act);
    if (rc) return rc;
    SB_HIP(dev_malloc(&L.act, (size_t)rows * L.M * net->esize));
    L.act_rows = rows;
  }
  return 0;
}

// After W or wmask of a layer with row lists has been written from outside (a restored checkpoint, say),
// one pass over W tells whether it is zero under every zero mask byte, i.e. whether the forward pass may
// walk the row lists right away.  Costs one read of W and a host round trip, once per such write.
template <typename T>
static int layer_check_masked(sb_net *net, Layer &L) {
  L.w_unchecked = false;
  if (!L.rows || L.w_masked) return 0;
  unsigned long long count = 0;
  SB_HIP(hipMemcpyAsync(net->d_unmasked, &count, sizeof(count), hipMemcpyHostToDevice, g_ctx.stream));
  int rc = launch_count_unmasked<T>(g_ctx.stream, (const T *)L.W, L.wmask, L.N, L.H, L.Mc, net->d_unmasked);
  if (rc) return rc;
  SB_HIP(hipMemcpyAsync(&count, net->d_unmasked, sizeof(count), hipMemcpyDeviceToHost, g_ctx.stream));
  SB_HIP(hipStreamSynchronize(g_ctx.stream));
  L.w_masked = count == 0;
  return 0;
}

// x_blocked: the same batch in blocks of 16 rows, or nullptr
template <typename T>
static int layer_forward(sb_net *net, Layer &L, const T *x, long B, const T *x_blocked = nullptr) {
  if (L.w_unchecked) {
    int rc = layer_check_masked<T>(net, L);
    if (rc) return rc;
  }
  if (L.rows && L.w_masked)
    return launch_forward_rows<T>(g_ctx.stream, (T *)L.act, x, (const T *)L.W, (const T *)L.bias, L.rows,
                                  L.row_cnt, L.rows_cap, B, L.N, L.H, L.Mc, x_blocked);
  return launch_forward<T>(g_ctx.stream, (T *)L.act, x, (const T *)L.W, (const T *)L.bias, B, L.N, L.H,
                           L.Mc, true);
}

// One training step of `L` on input x (and on y = its own activation or the labels), in the order of
// cpu_backend.py:13-15 (dense) and :29-52 (plastic).  W stays masked; on rewiring steps hypercolumn h
// is re-scored from the traces and its W columns rewritten under the new mask.
// next / next_bytes: what the step after this one reads first (its batch of inputs), or nullptr
template <typename T>
static int layer_train_step(Layer &L, const T *x, const T *y, long B, long h, const void *next = nullptr,
                            size_t next_bytes = 0) {
  hipStream_t st = g_ctx.stream;
  const T tau = (T)L.taupdt;
  const T cthr = (T)(L.taupdt / 2);
  int rc = 0;
  rc = launch_train_fused<T>(st, x, y, (T *)L.Cij, (T *)L.W, (const T *)L.Ci, (const T *)L.Cj,
                             (T *)L.Ci_alt, (T *)L.Cj_alt, L.plastic ? L.wmask : nullptr,
                             L.plastic ? 1 : 0, (T *)L.bias, (T *)L.kbi, B, L.N, L.H, L.Mc, tau, cthr,
                             (T)L.khalf, (T)L.pmin, (T)L.taubdt, L.w_masked, next, next_bytes);
  if (rc) return rc;
  std::swap(L.Ci, L.Ci_alt);
  std::swap(L.Cj, L.Cj_alt);
  // every entry of W has just been written under the mask
  if (L.plastic) L.w_masked = true, L.w_unchecked = false;
  if (L.plastic && h >= 0) {
    rc = launch_rewire<T>(st, L.wmask, (T *)L.W, (const T *)L.Ci, (const T *)L.Cj, (const T *)L.Cij, cthr, L.N,
                          L.H, L.Mc, h, 16, (T *)L.nom, L.csum, L.rows, L.row_cnt, L.rows_cap);
    // (a swap leaves the number of connected rows of the hypercolumn as it was, so its list still fits)
    if (rc) return rc;
  }
  return 0;
}

// After wmask has been replaced from the host copy `mask` [N, H]: (re)build the row lists when at most
// 70 % of the connections exist and the forward kernel over row lists takes the layer's shape, drop
// them otherwise.
template <typename T>
static int layer_mask_replaced(Layer &L, const uint8_t *mask) {
  L.w_masked = false;
  L.w_unchecked = true;
  std::vector<long> count((size_t)L.H, 0);
  for (long i = 0; i < L.N; i++)
    for (long h = 0; h < L.H; h++) count[(size_t)h] += mask[i * L.H + h] != 0;
  long total = 0, most = 0;
  for (long c : count) total += c, most = c > most ? c : most;
  // (the forward pass over row lists measured faster than the dense one up to a density of about 0.75)
  const bool sparse = 10 * total <= 7 * L.N * L.H && forward_rows_supported<T>((const T *)L.W, L.N, L.H, L.Mc);
  const long cap = (most + 15) / 16 * 16 + 16;
  if (!sparse || cap > L.rows_cap) {
    SB_HIP(hipStreamSynchronize(g_ctx.stream));
    void *r = L.rows, *c = L.row_cnt;
    int rc = free_dev(r) | free_dev(c);
    L.rows = nullptr; L.row_cnt = nullptr; L.rows_cap = 0;
    if (rc) return rc;
  }
  if (!sparse) return 0;
  if (!L.rows) {
    SB_HIP(dev_malloc((void **)&L.rows, (size_t)L.H * cap * sizeof(int)));
    SB_HIP(dev_malloc((void **)&L.row_cnt, (size_t)L.H * sizeof(int)));
    L.rows_cap = cap;
  }
  return launch_mask_rows(g_ctx.stream, L.rows, L.row_cnt, L.wmask, L.N, L.H, L.rows_cap, 0, L.H);
}

// Largest cache of frozen activations kept (bytes, both copies together): at most 16 GiB, and at most half of
// the device memory that is free when the cache is built; beyond it the activations are recomputed.
static bool frozen_cache_affordable(const sb_net *net, size_t bytes) {
  if (bytes > net->frozen_cache_limit) return false;
  size_t free_b = 0, total_b = 0;
  if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return bytes <= free_b / 2;
}

static int drop_frozen_cache(sb_net *net) {
  if (!net->Hc && !net->Hcp) {
    net->Hc_layer = -1;
    return 0;
  }
  SB_HIP(hipStreamSynchronize(g_ctx.stream));
  int rc = free_dev(net->Hc) | free_dev(net->Hcp);
  net->Hc_layer = -1;
  return rc;
}

// Activations of layer `upto` for all training samples in data-set order, in batches of maxB (the batch
// size the training steps use, so the same kernel variants run).
template <typename T>
static int build_frozen_cache(sb_net *net, int upto, long maxB) {
  const long Ns = net->Ns, Mo = net->layers[upto].M;
  int rc = drop_frozen_cache(net);
  if (rc) return rc;
  // without the memory for both copies the caller goes on uncached (Hc_layer stays -1): not an error
  if (dev_malloc(&net->Hc, (size_t)Ns * Mo * sizeof(T)) != hipSuccess ||
      dev_malloc(&net->Hcp, (size_t)Ns * Mo * sizeof(T)) != hipSuccess) {
    (void)hipGetLastError();
    net->Hcp = nullptr;
    if (net->Hc) (void)hipFree(net->Hc);
    net->Hc = nullptr;
    return 0;
  }
  for (long lo = 0; lo < Ns; lo += maxB) {
    const long B = lo + maxB <= Ns ? maxB : Ns - lo;
    const T *x = (const T *)net->X + lo * net->NF;
    for (int l = 0; l <= upto; l++) {
      if ((rc = layer_forward<T>(net, net->layers[l], x, B))) return rc;
      x = (const T *)net->layers[l].act;
    }
    SB_HIP(hipMemcpyAsync((T *)net->Hc + lo * Mo, x, (size_t)B * Mo * sizeof(T), hipMemcpyDeviceToDevice,
                          g_ctx.stream));
  }
  net->Hc_layer = upto;
  return 0;
}

template <typename T>
static int net_train_batches(sb_net *net, int layer, long maxB, const int64_t *h_sample_perm,
                             const int64_t *h_hc_perm, long epoch, long first_batch, long n_batches,
                             bool finalize) {
  hipStream_t st = g_ctx.stream;
  Layer &target = net->layers[layer];
  const bool last = layer + 1 == (int)net->layers.size();
  SB_REQUIRE(!last || net->Y, "the last layer trains on labels but none were given");
  SB_REQUIRE(!last || net->NC == target.M, "label width does not match the last layer");
  SB_REQUIRE(last || target.plastic, "a dense layer can only be trained as the last layer");
  SB_REQUIRE(net->layers[0].N == net->NF, "image width does not match the first layer");
  for (int l = 1; l <= layer; l++)
    SB_REQUIRE(net->layers[l].N == net->layers[l - 1].M, "layer widths do not chain");
  const long Ns = net->Ns;
  const long nb = (Ns + maxB - 1) / maxB;
  SB_REQUIRE(first_batch >= 0 && n_batches >= 0 && first_batch + n_batches <= nb, "batch range");
  int rc = ensure_act(net, maxB < Ns ? maxB : Ns);
  if (rc) return rc;
  const bool permute = first_batch == 0;  // a later range continues the epoch already laid out
  SB_REQUIRE(permute || net->Xp, "the epoch's first batches have not been run");
  // a training step of a layer below the last changes what the cache was computed from
  if (!last && (rc = drop_frozen_cache(net))) return rc;
  const long Mprev = layer > 0 ? net->layers[layer - 1].M : 0;
  const bool cache_fits = last && layer > 0 &&
                          (net->Hc_layer == layer - 1 || frozen_cache_affordable(net, 2 * (size_t)Ns * Mprev * sizeof(T)));
  if (permute) {
    SB_REQUIRE(h_sample_perm, "sample order missing");
    for (long r = 0; r < Ns; r++)
      SB_REQUIRE(h_sample_perm[r] >= 0 && h_sample_perm[r] < Ns, "sample index out of range");

    // images[idx, :] / labels[idx, :]  (_cpu_base_backend.py:258-260)
    if (!net->Xp) SB_HIP(dev_malloc(&net->Xp, (size_t)Ns * net->NF * net->esize));
    if (last && !net->Yp) SB_HIP(dev_malloc(&net->Yp, (size_t)Ns * net->NC * net->esize));
    SB_HIP(hipEventSynchronize(net->perm_copied));  // staging buffer free again
    std::memcpy(net->h_perm, h_sample_perm, (size_t)Ns * sizeof(int64_t));
    SB_HIP(hipMemcpyAsync(net->d_perm, net->h_perm, (size_t)Ns * sizeof(int64_t), hipMemcpyHostToDevice,
                          st));
    SB_HIP(hipEventRecord(net->perm_copied, st));
    // A first layer that walks row lists reads its input column by column: it gets the shuffled images a
    // second time, in blocks of 16 rows (batches must then start on block boundaries); one kernel writes
    // both copies from one read.
    if (net->layers[0].rows && maxB % 16 == 0) {
      if (!net->XpB) SB_HIP(dev_malloc(&net->XpB, (size_t)cdiv_l(Ns, 16) * 16 * net->NF * net->esize));
      if ((rc = launch_gather_rows_blocked<T>(st, (T *)net->XpB, (T *)net->Xp, (const T *)net->X, net->d_perm, Ns,
                                              net->NF)))
        return rc;
      net->XpB_batch = maxB;
    } else {
      if ((rc = launch_gather_rows<T>(st, (T *)net->Xp, (const T *)net->X, net->d_perm, Ns, net->NF)))
        return rc;
      net->XpB_batch = 0;
    }
    if (last)
      if ((rc = launch_gather_rows<T>(st, (T *)net->Yp, (const T *)net->Y, net->d_perm, Ns, net->NC)))
        return rc;
    if (cache_fits) {
      if (net->Hc_layer != layer - 1 && (rc = build_frozen_cache<T>(net, layer - 1, maxB))) return rc;
      if (net->Hc_layer == layer - 1 &&
          (rc = launch_gather_rows<T>(st, (T *)net->Hcp, (const T *)net->Hc, net->d_perm, Ns, Mprev)))
        return rc;
    } else if (last && (rc = drop_frozen_cache(net))) {
      return rc;
    }
  }
  const bool cached = cache_fits && net->Hc_layer == layer - 1;

  const long period = nb / (target.H + 1);  // _cpu_base_backend.py:297-299
  for (long i = first_batch; i < first_batch + n_batches; i++) {
    const long lo = i * maxB;
    const long B = (lo + maxB <= Ns) ? maxB : Ns - lo;
    const T *x = (const T *)net->Xp + lo * net->NF;
    const T *xb = net->XpB_batch == maxB ? (const T *)net->XpB + lo * net->NF : nullptr;  // lo % 16 == 0
    if (cached) {
      x = (const T *)net->Hcp + lo * Mprev;
    } else {
      for (int l = 0; l < layer; l++) {
        if ((rc = layer_forward<T>(net, net->layers[l], x, B, l == 0 ? xb : nullptr))) return rc;
        x = (const T *)net->layers[l].act;
      }
    }
    long h = -1;
    if (!last && epoch > 0 && period > 0 && i % period == 0) {
      const long slot = i / period;
      if (slot < target.H) {
        SB_REQUIRE(h_hc_perm, "hypercolumn order missing");
        h = h_hc_perm[slot];
        SB_REQUIRE(h >= 0 && h < target.H, "hypercolumn index out of range");
      }
    }
    if (last) {
      // the reference also evaluates the last layer's activation here and drops it
      // (_cpu_base_backend.py:290-295, 304-306); it has no effect on any state
      rc = layer_train_step<T>(target, x, (const T *)net->Yp + lo * net->NC, B, -1);
    } else {
      if ((rc = layer_forward<T>(net, target, x, B, layer == 0 ? xb : nullptr))) return rc;
      // The next step's images, when its forward pass is the dense one, which reads its input in step with W
      // and waits for every cold line (1568 -> 30 x 100, batch 128: 19.1 -> 15.9 us with the images found in the
      // memory-side cache instead of HBM; the pass over row lists gains 0.2 us, less than the extra workgroups
      // cost the training launch).
      const long nlo = lo + maxB;
      const bool more = layer == 0 && i + 1 < nb && !(target.rows && target.w_masked);
      const long nB = more ? (nlo + maxB <= Ns ? maxB : Ns - nlo) : 0;
      const T *nx = xb ? xb + maxB * net->NF : (const T *)net->Xp + nlo * net->NF;
      rc = layer_train_step<T>(target, x, (const T *)target.act, B, h, more ? nx : nullptr,
                               (size_t)nB * net->NF * sizeof(T));
    }
    if (rc) return rc;
  }
  // train_finalize, once per epoch (_cpu_base_backend.py:314; cpu_backend.py:17-18)
  if (finalize && !target.plastic)
    return launch_update_bias<T>(st, (T *)target.bias, (const T *)target.Cj, (T)(target.taupdt / 2),
                                 target.M);
  return 0;
}

template <typename T>
static int net_forward_batches(sb_net *net, const void *h_images, const void *h_labels, long n,
                               long NF, long NC, long maxB, int last_layer, void *h_act,
                               int64_t *correct, int32_t *h_pred) {
  hipStream_t st = g_ctx.stream;
  SB_REQUIRE(!net->layers.empty(), "network has no layers");
  SB_REQUIRE(last_layer >= 0 && last_layer < (int)net->layers.size(), "layer index out of range");
  SB_REQUIRE(net->layers[0].N == NF, "image width does not match the first layer");
  for (int l = 1; l <= last_layer; l++)
    SB_REQUIRE(net->layers[l].N == net->layers[l - 1].M, "layer widths do not chain");
  Layer &out = net->layers[last_layer];
  SB_REQUIRE(!h_labels || NC == out.M, "label width does not match the last layer");
  if (n == 0) return 0;
  int rc = ensure_act(net, maxB < n ? maxB : n);
  if (rc) return rc;
  // stream the set through HBM in chunks of whole batches (<= ~256 MiB of images at a time)
  long chunk = (256L << 20) / (long)(NF * sizeof(T));
  chunk = chunk / maxB * maxB;
  if (chunk < maxB) chunk = maxB;
  if (chunk > n) chunk = n;
  if ((rc = reuse_dev(net->ev_x, (size_t)chunk * NF * sizeof(T)))) return rc;
  // a first layer that walks row lists also gets every chunk in blocks of 16 rows (see net_train_batches)
  const bool blocked = net->layers[0].rows && maxB % 16 == 0;
  if (blocked && (rc = reuse_dev(net->ev_xb, (size_t)cdiv_l(chunk, 16) * 16 * NF * sizeof(T)))) return rc;
  if (h_labels && (rc = reuse_dev(net->ev_y, (size_t)chunk * NC * sizeof(T)))) return rc;
  if (h_pred && (rc = reuse_dev(net->ev_p, (size_t)chunk * sizeof(int32_t)))) return rc;
  void *const dX = net->ev_x.p, *const dY = net->ev_y.p, *const dXB = net->ev_xb.p;
  int32_t *const dP = (int32_t *)net->ev_p.p;
  if (h_labels) {
    unsigned long long zero = 0;
    SB_HIP(hipMemcpy(net->d_correct, &zero, sizeof(zero), hipMemcpyHostToDevice));
  }
  // Inside a chunk the images go up in pieces of whole batches (about 16 MiB) on a copy stream of their own,
  // through the pinned staging ring; the library's stream waits for a piece's event and works on its batches
  // while the next piece is on its way.
  if ((rc = stager_init())) return rc;
  hipStream_t up = g_stager.copy_stream;
  long piece = ((long)HostStager::kChunkBytes / (long)(NF * sizeof(T))) / maxB * maxB;
  if (piece < maxB) piece = maxB;
  for (long c0 = 0; c0 < n && !rc; c0 += chunk) {
    const long rows = (c0 + chunk <= n) ? chunk : n - c0;
    if (h_labels) {
      if ((rc = staged_upload(dY, (const T *)h_labels + c0 * NC, (size_t)rows * NC * sizeof(T), up))) break;
    }
    for (long lo = 0; lo < rows && !rc; lo += maxB) {
      if (lo % piece == 0) {  // the piece that starts here
        const long prows = lo + piece <= rows ? piece : rows - lo;
        if ((rc = staged_upload((T *)dX + lo * NF, (const T *)h_images + (c0 + lo) * NF,
                                (size_t)prows * NF * sizeof(T), up)))
          break;
        SB_HIP(hipEventRecord(g_stager.uploaded, up));
        SB_HIP(hipStreamWaitEvent(st, g_stager.uploaded, 0));
        // (pieces start on multiples of the batch size, which is a multiple of 16 where blocks are used)
        if (blocked)
          rc = launch_gather_rows_blocked<T>(st, (T *)dXB + lo * NF, (T *)nullptr, (const T *)dX + lo * NF, nullptr,
                                             prows, NF);
        if (rc) break;
      }
      const long B = (lo + maxB <= rows) ? maxB : rows - lo;
      const T *x = (const T *)dX + lo * NF;
      const T *xb = blocked ? (const T *)dXB + lo * NF : nullptr;
      const bool classify = h_labels || h_pred;
      for (int l = 0; l <= last_layer && !rc; l++) {
        Layer &L = net->layers[l];
        if (l == last_layer && classify && !L.plastic)
          // output layer: activation and classification (first maximal unit, comparison with the labels)
          rc = launch_forward_classify<T>(st, (T *)L.act, x, (const T *)L.W, (const T *)L.bias, B, L.N, L.H,
                                          L.Mc, true, h_labels ? (const T *)dY + lo * NC : nullptr,
                                          dP ? dP + lo : nullptr, net->d_correct);
        else
          rc = layer_forward<T>(net, L, x, B, l == 0 ? xb : nullptr);
        x = (const T *)L.act;
      }
      if (rc) break;
      if (classify && out.plastic)
        rc = launch_argmax_rows<T>(st, (const T *)out.act, h_labels ? (const T *)dY + lo * NC : nullptr,
                                   B, out.M, dP ? dP + lo : nullptr, net->d_correct);
      if (!rc && h_act)
        SB_HIP(hipMemcpyAsync((T *)h_act + (c0 + lo) * out.M, out.act, (size_t)B * out.M * sizeof(T),
                              hipMemcpyDeviceToHost, st));
    }
    if (!rc && h_pred) {
      SB_HIP(hipMemcpyAsync(h_pred + c0, dP, (size_t)rows * sizeof(int32_t), hipMemcpyDeviceToHost, st));
    }
    SB_HIP(hipStreamSynchronize(st));
  }
  if (!rc && h_labels && correct) {
    unsigned long long cnt = 0;
    SB_HIP(hipMemcpy(&cnt, net->d_correct, sizeof(cnt), hipMemcpyDeviceToHost));
    *correct = (int64_t)cnt;
  }
  if (rc) (void)hipStreamSynchronize(st);  // nothing in flight may still use the chunk buffers
  return rc;
}

// compute_activation / train_step of ONE layer on host arrays (the layer-level calls of the DSL)
template <typename T>
static int net_layer_activation(sb_net *net, int layer, const void *h_in, long rows, void *h_act) {
  Layer &L = net->layers[layer];
  int rc = ensure_act(net, rows);
  if (rc) return rc;
  ScopedDeviceBuffer bX;
  SB_HIP(dev_malloc(&bX.p, (size_t)rows * L.N * sizeof(T)));
  SB_HIP(hipMemcpy(bX.p, h_in, (size_t)rows * L.N * sizeof(T), hipMemcpyHostToDevice));
  rc = layer_forward<T>(net, L, (const T *)bX.p, rows);
  if (!rc) SB_HIP(hipMemcpyAsync(h_act, L.act, (size_t)rows * L.M * sizeof(T), hipMemcpyDeviceToHost, g_ctx.stream));
  SB_HIP(hipStreamSynchronize(g_ctx.stream));
  return rc;
}

template <typename T>
static int net_layer_train_step(sb_net *net, int layer, const void *h_in, const void *h_out, long rows, long h) {
  Layer &L = net->layers[layer];
  SB_REQUIRE(h < 0 || L.plastic, "only structural-plasticity layers rewire");
  SB_REQUIRE(h < L.H, "hypercolumn index out of range");
  int rc = drop_frozen_cache(net);  // the layer changes: what was computed from it is stale
  if (rc) return rc;
  ScopedDeviceBuffer bX, bY;
  SB_HIP(dev_malloc(&bX.p, (size_t)rows * L.N * sizeof(T)));
  SB_HIP(dev_malloc(&bY.p, (size_t)rows * L.M * sizeof(T)));
  SB_HIP(hipMemcpy(bX.p, h_in, (size_t)rows * L.N * sizeof(T), hipMemcpyHostToDevice));
  SB_HIP(hipMemcpy(bY.p, h_out, (size_t)rows * L.M * sizeof(T), hipMemcpyHostToDevice));
  rc = layer_train_step<T>(L, (const T *)bX.p, (const T *)bY.p, rows, h);
  SB_HIP(hipStreamSynchronize(g_ctx.stream));  // the staging buffers go out of scope
  return rc;
}

// Initial weights, bias and mask as the reference's GPU backend object draws them at construction
// (backend_full_cuda_internals.cu:151-155: weights ~ N(0, 0.1), bias ~ 0.1 U(0, 1); helpers_training.cu:10-32:
// mask bytes set with probability `density`, 0.1 there), from a generator seeded with `seed`.  Drawn on the
// host in pieces of at most 64 MiB and uploaded; synchronous.
template <typename T>
static int net_randomize_layer(sb_net *net, int layer, uint64_t seed, double density) {
  Layer &L = net->layers[layer];
  std::mt19937_64 gen(seed);
  std::normal_distribution<double> normal(0.0, 0.1);
  std::uniform_real_distribution<double> uniform(0.0, 1.0);
  const size_t nm = (size_t)L.N * L.M, piece = ((size_t)64 << 20) / sizeof(T);
  std::vector<T> buf(std::min(nm, piece));
  for (size_t lo = 0; lo < nm; lo += piece) {
    const size_t n = std::min(piece, nm - lo);
    for (size_t k = 0; k < n; k++) buf[k] = (T)normal(gen);
    SB_HIP(hipMemcpy((T *)L.W + lo, buf.data(), n * sizeof(T), hipMemcpyHostToDevice));
  }
  buf.resize((size_t)L.M);
  for (long j = 0; j < L.M; j++) buf[(size_t)j] = (T)(0.1 * uniform(gen));
  SB_HIP(hipMemcpy(L.bias, buf.data(), (size_t)L.M * sizeof(T), hipMemcpyHostToDevice));
  L.w_masked = false;
  L.w_unchecked = true;
  int rc = drop_frozen_cache(net);
  if (rc || !L.plastic) return rc;
  std::vector<uint8_t> mask((size_t)L.N * L.H);
  for (auto &b : mask) b = uniform(gen) < density ? 1 : 0;
  SB_HIP(hipMemcpy(L.wmask, mask.data(), mask.size(), hipMemcpyHostToDevice));
  return layer_mask_replaced<T>(L, mask.data());
}

struct StateRef {
  void *ptr;
  size_t bytes;
};

static int layer_state(sb_net *net, int layer, const char *name, StateRef &out) {
  SB_REQUIRE(net && name, "null pointer");
  SB_REQUIRE(layer >= 0 && layer < (int)net->layers.size(), "layer index out of range");
  Layer &L = net->layers[layer];
  const size_t e = net->esize;
  const std::string n(name);
  if (n == "weights") out = {L.W, (size_t)L.N * L.M * e};
  else if (n == "Cij") out = {L.Cij, (size_t)L.N * L.M * e};
  else if (n == "bias") out = {L.bias, (size_t)L.M * e};
  else if (n == "Cj") out = {L.Cj, (size_t)L.M * e};
  else if (n == "Ci") out = {L.Ci, (size_t)L.N * e};
  else if (n == "kbi" && L.plastic) out = {L.kbi, (size_t)L.M * e};
  else if (n == "wmask" && L.plastic) out = {L.wmask, (size_t)L.N * L.H};
  else {
    set_error("layer_state: unknown state array '" + n + "'");
    return SB_ERR_INVALID;
  }
  return 0;
}

// The C entry points whose host-side work allocates (vectors sized by the layer, the network object) run it
// through this: an exception must not cross the C boundary.
template <typename F>
static int no_throw(const char *where, F &&body) {
  try {
    return body();
  } catch (const std::bad_alloc &) {
    set_error(std::string(where) + ": out of host memory");
  } catch (const std::exception &e) {
    set_error(std::string(where) + ": " + e.what());
  }
  return SB_ERR_STATE;
}

}  // namespace sb

using namespace sb;

// ==================================================================================== C ABI: library
extern "C" {

int sb_abi_version(void) { return 1; }
const char *sb_last_error(void) { return g_error.c_str(); }

int sb_init(int device) {
  std::lock_guard<std::mutex> lock(g_ctx_mutex);
  if (g_ctx.ready) {
    if (g_ctx.device == device) return 0;
    set_error("sb_init: already initialised on another device");
    return SB_ERR_STATE;
  }
  int count = 0;
  SB_HIP(hipGetDeviceCount(&count));
  SB_REQUIRE(device >= 0 && device < count, "no such device");
  SB_HIP(hipSetDevice(device));
  hipDeviceProp_t prop;
  SB_HIP(hipGetDeviceProperties(&prop, device));
  if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    set_error(std::string("sb_init: this library is built for gfx950 only, device is ") + prop.gcnArchName);
    return SB_ERR_UNSUPPORTED;
  }
  // device address of the static scratch array on this device (the device is current here)
  void *scratch_ptr = nullptr;
  SB_HIP(hipGetSymbolAddress(&scratch_ptr, HIP_SYMBOL(scratch)));
  SB_REQUIRE(scratch_ptr, "no device address for the static scratch array");
  SB_HIP(hipStreamCreate(&g_ctx.stream));
  g_ctx.noalloc_scratch = scratch_ptr;
  g_ctx.device = device;
  g_ctx.ready = true;
  return 0;
}

int sb_shutdown(void) {
  std::lock_guard<std::mutex> lock(g_ctx_mutex);
  if (!g_ctx.ready) return 0;
  SB_HIP(hipStreamSynchronize(g_ctx.stream));
  if (g_ctx.mask_nom) SB_HIP(hipFree(g_ctx.mask_nom));
  if (g_ctx.mask_csum) SB_HIP(hipFree(g_ctx.mask_csum));
  if (g_ctx.trace_next) SB_HIP(hipFree(g_ctx.trace_next));
  stager_release();
  SB_HIP(hipStreamDestroy(g_ctx.stream));
  g_ctx = Context();
  return 0;
}

int sb_sync(void) {
  SB_READY();
  SB_HIP(hipStreamSynchronize(g_ctx.stream));
  return 0;
}

long sb_allocation_calls(void) { return g_allocation_calls; }

void *sb_stream(void) { return g_ctx.ready ? (void *)g_ctx.stream : nullptr; }

int sb_malloc(void **d_ptr, size_t bytes) {
  SB_READY();
  SB_REQUIRE(d_ptr, "null pointer");
  SB_HIP(dev_malloc(d_ptr, bytes ? bytes : 1));
  return 0;
}
int sb_free(void *d_ptr) {
  SB_READY();
  if (!d_ptr) return 0;
  SB_HIP(hipStreamSynchronize(g_ctx.stream));
  SB_HIP(hipFree(d_ptr));
  return 0;
}
int sb_memcpy_h2d(void *d_dst, const void *h_src, size_t bytes) {
  SB_READY();
  if (!bytes) return 0;
  SB_REQUIRE(d_dst && h_src, "null pointer");
  SB_HIP(hipMemcpyAsync(d_dst, h_src, bytes, hipMemcpyHostToDevice, g_ctx.stream));
  SB_HIP(hipStreamSynchronize(g_ctx.stream));
  return 0;
}
int sb_memcpy_d2h(void *h_dst, const void *d_src, size_t bytes) {
  SB_READY();
  if (!bytes) return 0;
  SB_REQUIRE(h_dst && d_src, "null pointer");
  SB_HIP(hipMemcpyAsync(h_dst, d_src, bytes, hipMemcpyDeviceToHost, g_ctx.stream));
  SB_HIP(hipStreamSynchronize(g_ctx.stream));
  return 0;
}
int sb_memcpy_d2d(void *d_dst, const void *d_src, size_t bytes) {
  SB_READY();
  if (!bytes) return 0;
  SB_REQUIRE(d_dst && d_src, "null pointer");
  SB_HIP(hipMemcpyAsync(d_dst, d_src, bytes, hipMemcpyDeviceToDevice, g_ctx.stream));
  return 0;
}
int sb_mask_rows(int *d_rows, int *d_row_cnt, const uint8_t *d_wmask, long N, long H, long cap) {
  SB_READY();
  return launch_mask_rows(g_ctx.stream, d_rows, d_row_cnt, d_wmask, N, H, cap, 0, H);
}
int sb_fill_bytes(void *d_dst, int value, size_t bytes) {
  SB_READY();
  return launch_fill_bytes(g_ctx.stream, d_dst, value, bytes);
}

// ============================================================================ C ABI: per-kernel calls
#define SB_DEFINE_KERNEL_API(SFX, T)                                                                   \
  int sb_update_state_##SFX(T *act, const T *x, const T *W, const T *bias, long B, long N, long M) {   \
    SB_READY();                                                                                        \
    return launch_forward<T>(g_ctx.stream, act, x, W, bias, B, N, 1, M, false);                        \
  }                                                                                                    \
  int sb_softmax_minicolumns_##SFX(T *act, long B, long H, long Mc) {                                  \
    SB_READY();                                                                                        \
    return launch_softmax<T>(g_ctx.stream, act, B, H, Mc);                                             \
  }                                                                                                    \
  int sb_compute_activation_##SFX(T *act, const T *x, const T *W, const T *bias, long B, long N,       \
                                  long H, long Mc) {                                                   \
    SB_READY();                                                                                        \
    SB_REQUIRE(B > 0 && N > 0 && H > 0 && Mc > 0, "sizes must be positive");                           \
    return launch_forward<T>(g_ctx.stream, act, x, W, bias, B, N, H, Mc, true);                        \
  }                                                                                                    \
  int sb_compute_activation_rows_##SFX(T *act, const T *x, const T *W, const T *bias, const int *rows, \
                                       const int *row_cnt, long cap, long B, long N, long H, long Mc,  \
                                       const T *x_blocked) {                                           \
    SB_READY();                                                                                        \
    return launch_forward_rows<T>(g_ctx.stream, act, x, W, bias, rows, row_cnt, cap, B, N, H, Mc,      \
                                  x_blocked);                                                          \
  }                                                                                                    \
  int sb_rows_in_blocks_##SFX(T *dst, const T *src, long rows, long cols) {                            \
    SB_READY();                                                                                        \
    return launch_gather_rows_blocked<T>(g_ctx.stream, dst, (T *)nullptr, src, nullptr, rows, cols);   \
  }                                                                                                    \
  int sb_update_weights_##SFX(T *Ci, T *Cj, T *Cij, const T *a_i, const T *a_o, T taupdt, T *W,        \
                              T cthr, long B, long N, long M) {                                        \
    SB_READY();                                                                                        \
    return train_in_place<T>(a_i, a_o, Cij, W, Ci, Cj, nullptr, 0, nullptr, nullptr, B, N, 1, M, taupdt, \
                             cthr, T(0), T(0), T(0));                                                  \
  }                                                                                                    \
  int sb_update_counters_##SFX(T *Ci, T *Cj, T *Cij, const T *a_i, const T *a_o, T taupdt, long B,     \
                               long N, long M) {                                                       \
    SB_READY();                                                                                        \
    return train_in_place<T>(a_i, a_o, Cij, (T *)nullptr, Ci, Cj, nullptr, 0, nullptr, nullptr, B, N, 1, M, \
                             taupdt, (T)(taupdt / 2), T(0), T(0), T(0));                               \
  }                                                                                                    \
  int sb_weights_from_counters_##SFX(T *W, const T *Ci, const T *Cj, const T *Cij, T cthr, long N,     \
                                     long M) {                                                         \
    SB_READY();                                                                                        \
    return launch_weights_from_traces<T>(g_ctx.stream, W, Ci, Cj, Cij, nullptr, cthr, N, 1, M, false); \
  }                                                                                                    \
  int sb_weights_masked_from_counters_##SFX(T *W, const T *Ci, const T *Cj, const T *Cij,              \
                                            const uint8_t *wmask, T cthr, long N, long H, long Mc) {   \
    SB_READY();                                                                                        \
    SB_REQUIRE(wmask, "null pointer");                                                                 \
    return launch_weights_from_traces<T>(g_ctx.stream, W, Ci, Cj, Cij, wmask, cthr, N, H, Mc, false);  \
  }                                                                                                    \
  int sb_add_bias_##SFX(T *act, const T *bias, long B, long M) {                                       \
    SB_READY();                                                                                        \
    return launch_add_bias<T>(g_ctx.stream, act, bias, B, M);                                          \
  }                                                                                                    \
  int sb_update_bias_##SFX(T *bias, const T *Cj, T cthr, long M) {                                     \
    SB_READY();                                                                                        \
    return launch_update_bias<T>(g_ctx.stream, bias, Cj, cthr, M);                                     \
  }                                                                                                    \
  int sb_update_bias_regularized_##SFX(T *bias, T *kbi, const T *Cj, T cthr, T khalf, T pmin,          \
                                       T taubdt, long M) {                                             \
    SB_READY();                                                                                        \
    return launch_update_bias_regularized<T>(g_ctx.stream, bias, kbi, Cj, cthr, khalf, pmin, taubdt,   \
                                             M);                                                       \
  }                                                                                                    \
  int sb_update_mask_##SFX(uint8_t *wmask, const T *W, const T *Ci, const T *Cj, const T *Cij,         \
                           T cthr, long N, long H, long Mc, long h, long iterations) {                 \
    SB_READY();                                                                                        \
    SB_REQUIRE(W, "null pointer");                                                                     \
    SB_REQUIRE(N > 0, "sizes must be positive");                                                       \
    int rc = ensure_mask_scratch(N);                                                                   \
    if (rc) return rc;                                                                                 \
    return launch_update_mask<T>(g_ctx.stream, wmask, W, Ci, Cj, Cij, cthr, N, H, Mc, h, iterations,   \
                                 (T *)g_ctx.mask_nom, g_ctx.mask_csum);                                \
  }                                                                                                    \
  int sb_apply_mask_##SFX(T *W, const uint8_t *wmask, long N, long H, long Mc) {                       \
    SB_READY();                                                                                        \
    return launch_apply_mask<T>(g_ctx.stream, W, wmask, N, H, Mc);                                     \
  }                                                                                                    \
  int sb_argmax_rows_##SFX(const T *act, long B, long M, int32_t *pred) {                              \
    SB_READY();                                                                                        \
    SB_REQUIRE(pred, "null pointer");                                                                  \
    return launch_argmax_rows<T>(g_ctx.stream, act, nullptr, B, M, pred, nullptr);                     \
  }                                                                                                    \
  int sb_plastic_train_step_##SFX(T *W, T *bias, T *Ci, T *Cj, T *Cij, T *kbi, uint8_t *wmask,         \
                                  const T *x, const T *y, long B, long N, long H, long Mc, T taupdt,   \
                                  T khalf, T pmin, T taubdt, long h) {                                 \
    SB_READY();                                                                                        \
    SB_REQUIRE(W && bias && Ci && Cj && Cij && kbi && wmask && x && y, "null pointer");                \
    SB_REQUIRE(N > 0 && H > 0 && Mc > 0, "sizes must be positive");                                    \
    SB_REQUIRE(h < H, "hypercolumn index out of range");                                               \
    const T cthr = (T)((double)taupdt / 2);                                                            \
    int rc = train_in_place<T>(x, y, Cij, W, Ci, Cj, wmask, 1, bias, kbi, B, N, H, Mc, taupdt, cthr,     \
                               khalf, pmin, taubdt);                                                   \
    if (rc || h < 0) return rc;                                                                        \
    if ((rc = ensure_mask_scratch(N))) return rc;                                                      \
    return launch_rewire<T>(g_ctx.stream, wmask, W, Ci, Cj, Cij, cthr, N, H, Mc, h, 16,                \
                            (T *)g_ctx.mask_nom, g_ctx.mask_csum, nullptr, nullptr, 0);                \
  }

SB_DEFINE_KERNEL_API(f32, float)
SB_DEFINE_KERNEL_API(f64, double)

// sb_update_weights_f32 for callers that cannot allocate: the new Ci / Cj go through the static scratch
// array (every element the copies read is written by the kernel first, so nothing needs clearing).  No
// hipMalloc / hipFree on this path; the event brackets of sb_profile_start would create events, so the
// call is refused while they are on.
int sb_update_weights_noalloc_f32(float *Ci, float *Cj, float *Cij, const float *a_i, const float *a_o,
                                  float taupdt, float *W, float cthr, long B, long N, long M) {
  SB_READY();
  SB_REQUIRE(N > 0 && M > 0, "sizes must be positive");
  if (N + M > (long)SB_NOALLOC_MAX_UNITS) {
    set_error("sb_update_weights_noalloc_f32: N + M = " + std::to_string(N + M) + " exceeds SB_NOALLOC_MAX_UNITS = " +
              std::to_string((long)SB_NOALLOC_MAX_UNITS) + "; use sb_update_weights_f32");
    return SB_ERR_UNSUPPORTED;
  }
  if (g_prof_on) {
    set_error("sb_update_weights_noalloc_f32: not available between sb_profile_start and sb_profile_stop");
    return SB_ERR_STATE;
  }
  return train_in_place<float>(a_i, a_o, Cij, W, Ci, Cj, nullptr, 0, nullptr, nullptr, B, N, 1, M, taupdt, cthr,
                               0.f, 0.f, 0.f, (float *)g_ctx.noalloc_scratch);
}

// ================================================================================== C ABI: network
int sb_net_create(sb_net **net, int dtype) {
  SB_READY();
  SB_REQUIRE(net, "null pointer");
  SB_REQUIRE(dtype == SB_F32 || dtype == SB_F64, "dtype must be SB_F32 or SB_F64");
  sb_net *n = new (std::nothrow) sb_net();
  if (!n) {
    set_error("sb_net_create: out of host memory");
    return SB_ERR_STATE;
  }
  n->dtype = dtype;
  n->esize = dtype == SB_F32 ? 4 : 8;
  hipError_t e = dev_malloc((void **)&n->d_correct, sizeof(unsigned long long));
  if (e == hipSuccess) e = dev_malloc((void **)&n->d_unmasked, sizeof(unsigned long long));
  if (e == hipSuccess) e = (g_allocation_calls++, hipEventCreateWithFlags(&n->perm_copied, hipEventDisableTiming));
  if (e != hipSuccess) {
    if (n->d_correct) (void)hipFree(n->d_correct);
    if (n->d_unmasked) (void)hipFree(n->d_unmasked);
    delete n;
    return hip_fail(e, "sb_net_create", __FILE__, __LINE__);
  }
  *net = n;
  return 0;
}

int sb_net_training_done(sb_net *net) {
  SB_READY();
  SB_REQUIRE(net, "null pointer");
  SB_HIP(hipStreamSynchronize(g_ctx.stream));
  int rc = 0;
  void *p = net->d_perm;
  rc |= free_dev(net->X); rc |= free_dev(net->Y); rc |= free_dev(net->Xp); rc |= free_dev(net->Yp);
  rc |= free_dev(net->XpB);
  net->XpB_batch = 0;
  rc |= free_dev(net->Hc); rc |= free_dev(net->Hcp);
  net->Hc_layer = -1;
  rc |= free_dev(p);
  net->d_perm = nullptr;
  if (net->h_perm) SB_HIP(hipHostFree(net->h_perm));
  net->h_perm = nullptr;
  net->Ns = net->NF = net->NC = 0;
  return rc;
}

int sb_net_destroy(sb_net *net) {
  SB_READY();
  if (!net) return 0;
  int rc = sb_net_training_done(net);
  for (auto &L : net->layers) rc |= layer_free(L);
  rc |= free_dev(net->ev_x.p); rc |= free_dev(net->ev_xb.p); rc |= free_dev(net->ev_y.p); rc |= free_dev(net->ev_p.p);
  if (net->d_correct) SB_HIP(hipFree(net->d_correct));
  if (net->d_unmasked) SB_HIP(hipFree(net->d_unmasked));
  if (net->perm_copied) SB_HIP(hipEventDestroy(net->perm_copied));
  delete net;
  return rc;
}

static int add_layer(sb_net *net, bool plastic, long n_inputs, long H, long Mc, double taupdt,
                     double pmin, double khalf, double taubdt, double ci0, double cj0, double cij0) {
  SB_READY();
  SB_REQUIRE(net, "null pointer");
  SB_REQUIRE(n_inputs > 0 && H > 0 && Mc > 0, "sizes must be positive");
  SB_REQUIRE(n_inputs < (1L << 31) && H * Mc < (1L << 31), "dimension too large");
  Layer L;
  L.plastic = plastic;
  L.N = n_inputs; L.H = H; L.Mc = Mc; L.M = H * Mc;
  L.taupdt = taupdt; L.pmin = pmin; L.khalf = khalf; L.taubdt = taubdt;
  int rc = net->dtype == SB_F32 ? layer_alloc<float>(L, (float)ci0, (float)cj0, (float)cij0)
                                : layer_alloc<double>(L, ci0, cj0, cij0);
  if (rc) {
    layer_free(L);
    return rc;
  }
  net->layers.push_back(L);
  return (int)net->layers.size() - 1;
}

int sb_net_add_dense_layer(sb_net *net, long n_inputs, long hypercolumns, long minicolumns,
                           double taupdt, double initial_Ci, double initial_Cj, double initial_Cij) {
  return no_throw("sb_net_add_dense_layer", [&] {
    return add_layer(net, false, n_inputs, hypercolumns, minicolumns, taupdt, 0, 0, 0, initial_Ci, initial_Cj,
                     initial_Cij);
  });
}

int sb_net_add_plastic_layer(sb_net *net, long n_inputs, long hypercolumns, long minicolumns,
                             double taupdt, double pmin, double khalf, double taubdt,
                             double initial_Ci, double initial_Cj, double initial_Cij) {
  return no_throw("sb_net_add_plastic_layer", [&] {
    return add_layer(net, true, n_inputs, hypercolumns, minicolumns, taupdt, pmin, khalf, taubdt, initial_Ci,
                     initial_Cj, initial_Cij);
  });
}

int sb_net_set_layer_state(sb_net *net, int layer, const char *name, const void *h_src, size_t bytes) {
  SB_READY();
  StateRef s{};
  int rc = layer_state(net, layer, name, s);
  if (rc) return rc;
  SB_REQUIRE(h_src, "null pointer");
  SB_REQUIRE(bytes == s.bytes, "size mismatch");
  rc = sb_memcpy_h2d(s.ptr, h_src, bytes);
  if (rc) return rc;
  if ((rc = drop_frozen_cache(net))) return rc;  // (whatever layer: the cache is cheap to rebuild)
  Layer &L = net->layers[layer];
  if (s.ptr == L.W) L.w_masked = false, L.w_unchecked = true;
  if (s.ptr == L.wmask)
    return no_throw("sb_net_set_layer_state", [&] {
      return net->dtype == SB_F32 ? layer_mask_replaced<float>(L, (const uint8_t *)h_src)
                                  : layer_mask_replaced<double>(L, (const uint8_t *)h_src);
    });
  return 0;
}

int sb_net_get_layer_state(sb_net *net, int layer, const char *name, void *h_dst, size_t bytes) {
  SB_READY();
  StateRef s{};
  int rc = layer_state(net, layer, name, s);
  if (rc) return rc;
  SB_REQUIRE(h_dst, "null pointer");
  SB_REQUIRE(bytes == s.bytes, "size mismatch");
  return sb_memcpy_d2h(h_dst, s.ptr, bytes);
}

int sb_net_randomize_layer(sb_net *net, int layer, uint64_t seed, double density) {
  SB_READY();
  SB_REQUIRE(net, "null pointer");
  SB_REQUIRE(layer >= 0 && layer < (int)net->layers.size(), "layer index out of range");
  SB_REQUIRE(density >= 0.0, "density must be non-negative");
  SB_HIP(hipStreamSynchronize(g_ctx.stream));
  return no_throw("sb_net_randomize_layer", [&] {
    return net->dtype == SB_F32 ? net_randomize_layer<float>(net, layer, seed, density)
                                : net_randomize_layer<double>(net, layer, seed, density);
  });
}

int sb_net_set_frozen_cache_limit(sb_net *net, size_t bytes) {
  SB_READY();
  SB_REQUIRE(net, "null pointer");
  net->frozen_cache_limit = bytes;
  if (net->Hc && 2 * (size_t)net->Ns * (size_t)net->layers[net->Hc_layer].M * net->esize > bytes)
    return drop_frozen_cache(net);
  return 0;
}

int sb_net_set_training_data(sb_net *net, const void *h_images, const void *h_labels, long n_samples,
                             long n_features, long n_classes) {
  SB_READY();
  SB_REQUIRE(net && h_images, "null pointer");
  SB_REQUIRE(n_samples > 0 && n_features > 0, "sizes must be positive");
  SB_REQUIRE(!h_labels || n_classes > 0, "sizes must be positive");
  int rc = sb_net_training_done(net);
  if (rc) return rc;
  const size_t xb = (size_t)n_samples * n_features * net->esize;
  SB_HIP(dev_malloc(&net->X, xb));
  if ((rc = staged_upload(net->X, h_images, xb, g_ctx.stream))) return rc;
  if (h_labels) {
    const size_t yb = (size_t)n_samples * n_classes * net->esize;
    SB_HIP(dev_malloc(&net->Y, yb));
    if ((rc = staged_upload(net->Y, h_labels, yb, g_ctx.stream))) return rc;
  }
  SB_HIP(dev_malloc((void **)&net->d_perm, (size_t)n_samples * sizeof(int64_t)));
  g_allocation_calls++;
  SB_HIP(hipHostMalloc((void **)&net->h_perm, (size_t)n_samples * sizeof(int64_t), hipHostMallocDefault));
  SB_HIP(hipEventRecord(net->perm_copied, g_ctx.stream));
  net->Ns = n_samples;
  net->NF = n_features;
  net->NC = h_labels ? n_classes : 0;
  return 0;
}

int sb_net_train_batches(sb_net *net, int layer, long maximal_batch_size,
                         const int64_t *h_sample_perm, const int64_t *h_hc_perm, long epoch_index,
                         long first_batch, long n_batches, int finalize) {
  SB_READY();
  SB_REQUIRE(net, "null pointer");
  if (!net->X) {
    set_error("sb_net_train_batches: no training data (call sb_net_set_training_data)");
    return SB_ERR_STATE;
  }
  SB_REQUIRE(layer >= 0 && layer < (int)net->layers.size(), "layer index out of range");
  SB_REQUIRE(maximal_batch_size > 0, "batch size must be positive");
  SB_REQUIRE(epoch_index >= 0, "epoch index must be non-negative");
  return net->dtype == SB_F32
             ? net_train_batches<float>(net, layer, maximal_batch_size, h_sample_perm, h_hc_perm,
                                        epoch_index, first_batch, n_batches, finalize != 0)
             : net_train_batches<double>(net, layer, maximal_batch_size, h_sample_perm, h_hc_perm,
                                         epoch_index, first_batch, n_batches, finalize != 0);
}

int sb_net_train_epoch(sb_net *net, int layer, long maximal_batch_size, const int64_t *h_sample_perm,
                       const int64_t *h_hc_perm, long epoch_index) {
  SB_READY();
  SB_REQUIRE(net && h_sample_perm, "null pointer");
  SB_REQUIRE(maximal_batch_size > 0, "batch size must be positive");
  const long nb = net->Ns > 0 ? (net->Ns + maximal_batch_size - 1) / maximal_batch_size : 0;
  return sb_net_train_batches(net, layer, maximal_batch_size, h_sample_perm, h_hc_perm, epoch_index, 0,
                              nb, 1);
}

// Matrix-core probe (see k_mfma_probe); *flops receives the floating-point operations of the launch.
static int mfma_probe(int dtype, long workgroups, long iters, double *flops) {
  SB_READY();
  SB_REQUIRE(dtype == SB_F32 || dtype == SB_F64 || dtype == SB_PROBE_F64_4X4X4,
             "dtype must be SB_F32, SB_F64 or SB_PROBE_F64_4X4X4");
  int rc = ensure_trace_scratch(1);
  if (rc) return rc;
  if (dtype == SB_PROBE_F64_4X4X4) {
    rc = launch_mfma_probe_f64_4x4x4(g_ctx.stream, (double *)g_ctx.trace_next, workgroups, iters);
    if (!rc && flops) *flops = (double)workgroups * 4.0 * (double)iters * 16.0 * 2.0 * 4 * 4 * 4 * 4;
    return rc;
  }
  rc = dtype == SB_F32 ? launch_mfma_probe<float>(g_ctx.stream, (float *)g_ctx.trace_next, workgroups, iters)
                       : launch_mfma_probe<double>(g_ctx.stream, (double *)g_ctx.trace_next, workgroups, iters);
  if (!rc && flops) *flops = (double)workgroups * 4.0 * (double)iters * 8.0 * 2.0 * 16 * 16 * 4;
  return rc;
}
int sb_probe_mfma(int dtype, long workgroups, long iters, double *flops) {
  return mfma_probe(dtype, workgroups, iters, flops);
}

int sb_net_layer_activation(sb_net *net, int layer, const void *h_inputs, long n_rows, void *h_act) {
  SB_READY();
  SB_REQUIRE(net && h_inputs && h_act, "null pointer");
  SB_REQUIRE(layer >= 0 && layer < (int)net->layers.size(), "layer index out of range");
  SB_REQUIRE(n_rows > 0, "sizes must be positive");
  return net->dtype == SB_F32 ? net_layer_activation<float>(net, layer, h_inputs, n_rows, h_act)
                              : net_layer_activation<double>(net, layer, h_inputs, n_rows, h_act);
}

int sb_net_layer_train_step(sb_net *net, int layer, const void *h_inputs, const void *h_outputs, long n_rows,
                            long hypercolumn) {
  SB_READY();
  SB_REQUIRE(net && h_inputs && h_outputs, "null pointer");
  SB_REQUIRE(layer >= 0 && layer < (int)net->layers.size(), "layer index out of range");
  SB_REQUIRE(n_rows > 0, "sizes must be positive");
  return net->dtype == SB_F32
             ? net_layer_train_step<float>(net, layer, h_inputs, h_outputs, n_rows, hypercolumn)
             : net_layer_train_step<double>(net, layer, h_inputs, h_outputs, n_rows, hypercolumn);
}

int sb_net_layer_train_finalize(sb_net *net, int layer) {
  SB_READY();
  SB_REQUIRE(net, "null pointer");
  SB_REQUIRE(layer >= 0 && layer < (int)net->layers.size(), "layer index out of range");
  Layer &L = net->layers[layer];
  if (L.plastic) return 0;  // _cpu_base_backend.py:171-172
  int rc = drop_frozen_cache(net);
  if (rc) return rc;
  return net->dtype == SB_F32
             ? launch_update_bias<float>(g_ctx.stream, (float *)L.bias, (const float *)L.Cj, (float)(L.taupdt / 2), L.M)
             : launch_update_bias<double>(g_ctx.stream, (double *)L.bias, (const double *)L.Cj, L.taupdt / 2, L.M);
}

int sb_profile_start(void) {
  SB_READY();
  SB_HIP(hipStreamSynchronize(g_ctx.stream));
  for (auto &r : g_prof_records) {
    g_prof_pool.push_back(r.start);
    g_prof_pool.push_back(r.stop);
  }
  g_prof_records.clear();
  for (int k = 0; k < K_COUNT; k++) {
    g_prof_ms[k] = 0;
    g_prof_launches[k] = 0;
  }
  g_prof_carry = std::getenv("ROCPROF_OUTPUT_PATH") == nullptr;
  // what a bracket costs at most: median elapsed time of event pairs with nothing in between (reported
  // by sb_profile_bracket_overhead_us; the per-kernel sums stay raw)
  {
    constexpr int kPairs = 33;
    hipEvent_t ev[2 * kPairs];
    for (auto &e : ev) e = prof_event();
    for (int i = 0; i < kPairs; i++) {
      if (!ev[2 * i] || !ev[2 * i + 1]) continue;
      SB_HIP(hipEventRecord(ev[2 * i], g_ctx.stream));
      SB_HIP(hipEventRecord(ev[2 * i + 1], g_ctx.stream));
    }
    SB_HIP(hipStreamSynchronize(g_ctx.stream));
    std::vector<float> gaps;
    for (int i = 0; i < kPairs; i++) {
      float ms = 0;
      if (ev[2 * i] && ev[2 * i + 1] && hipEventElapsedTime(&ms, ev[2 * i], ev[2 * i + 1]) == hipSuccess)
        gaps.push_back(ms);
    }
    for (auto &e : ev)
      if (e) g_prof_pool.push_back(e);
    std::sort(gaps.begin(), gaps.end());
    g_prof_overhead_ms = gaps.empty() ? 0.0 : gaps[gaps.size() / 2];
  }
  g_prof_on = true;
  return 0;
}

int sb_profile_stop(void) {
  SB_READY();
  g_prof_on = false;
  SB_HIP(hipStreamSynchronize(g_ctx.stream));
  for (auto &r : g_prof_records) {
    float ms = 0;
    SB_HIP(hipEventElapsedTime(&ms, r.start, r.stop));
    g_prof_ms[r.id] += ms;
    g_prof_launches[r.id] += 1;
    g_prof_pool.push_back(r.start);
    g_prof_pool.push_back(r.stop);
  }
  g_prof_records.clear();
  return 0;
}

int sb_profile_kernels(void) { return K_COUNT; }

double sb_profile_bracket_overhead_us(void) { return 1e3 * g_prof_overhead_ms; }

const char *sb_profile_kernel_name(int kernel) { return kernel_name(kernel); }

int sb_profile_kernel_carried(int kernel) { return kernel >= 0 && kernel < K_COUNT && prof_carried(kernel) ? 1 : 0; }

int sb_profile_get(int kernel, double *total_ms, long *launches) {
  SB_REQUIRE(kernel >= 0 && kernel < K_COUNT && total_ms && launches, "bad argument");
  *total_ms = g_prof_ms[kernel];
  *launches = g_prof_launches[kernel];
  return 0;
}

int sb_net_evaluate(sb_net *net, const void *h_images, const void *h_labels, long n_samples,
                    long n_features, long n_classes, long maximal_batch_size, int64_t *correct,
                    int64_t *total, int32_t *h_pred) {
  SB_READY();
  SB_REQUIRE(net && h_images && h_labels && correct && total, "null pointer");
  SB_REQUIRE(n_samples >= 0 && n_features > 0 && n_classes > 0 && maximal_batch_size > 0, "bad sizes");
  *correct = 0;
  *total = n_samples;
  const int last = (int)net->layers.size() - 1;
  return net->dtype == SB_F32
             ? net_forward_batches<float>(net, h_images, h_labels, n_samples, n_features, n_classes,
                                          maximal_batch_size, last, nullptr, correct, h_pred)
             : net_forward_batches<double>(net, h_images, h_labels, n_samples, n_features, n_classes,
                                           maximal_batch_size, last, nullptr, correct, h_pred);
}

int sb_net_predict(sb_net *net, const void *h_images, long n_samples, long n_features,
                   long maximal_batch_size, int32_t *h_pred) {
  SB_READY();
  SB_REQUIRE(net && h_images && h_pred, "null pointer");
  SB_REQUIRE(n_samples >= 0 && n_features > 0 && maximal_batch_size > 0, "bad sizes");
  const int last = (int)net->layers.size() - 1;
  return net->dtype == SB_F32
             ? net_forward_batches<float>(net, h_images, nullptr, n_samples, n_features, 0,
                                          maximal_batch_size, last, nullptr, nullptr, h_pred)
             : net_forward_batches<double>(net, h_images, nullptr, n_samples, n_features, 0,
                                           maximal_batch_size, last, nullptr, nullptr, h_pred);
}

int sb_net_forward(sb_net *net, const void *h_images, long n_rows, long n_features, int last_layer,
                   long maximal_batch_size, void *h_act) {
  SB_READY();
  SB_REQUIRE(net && h_images && h_act, "null pointer");
  SB_REQUIRE(n_rows >= 0 && n_features > 0 && maximal_batch_size > 0, "bad sizes");
  return net->dtype == SB_F32
             ? net_forward_batches<float>(net, h_images, nullptr, n_rows, n_features, 0,
                                          maximal_batch_size, last_layer, h_act, nullptr, nullptr)
             : net_forward_batches<double>(net, h_images, nullptr, n_rows, n_features, 0,
                                           maximal_batch_size, last_layer, h_act, nullptr, nullptr);
}

}  // extern "C"
