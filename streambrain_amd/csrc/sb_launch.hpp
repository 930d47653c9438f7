// Host-side launchers: shape checks, kernel-variant selection and grid computation for every kernel.
// All launches go to the stream handed in; nothing here synchronises.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

namespace sb {

// Scalars of one layer narrowed to the element type the way the reference's call boundary does it:
// Python float64 -> REAL at the pybind call (omp.cc:362-365,400-402,419-422), cthr = taupdt/2 formed in
// float64 first (cpu_backend.py:15,31), 1-taupdt formed in double and narrowed (omp.cc:101), cthr^4 by
// repeated multiplication in REAL (omp.cc:102).
template <typename T>
struct TraceScalars {
  T tau, omt, cthr, cthr4;
  static TraceScalars from(T taupdt, T cthr_) {
    TraceScalars s;
    s.tau = taupdt;
    s.omt = (T)(1.0 - (double)taupdt);
    s.cthr = cthr_;
    volatile T c2 = cthr_ * cthr_;
    volatile T c3 = c2 * cthr_;
    s.cthr4 = c3 * cthr_;
    return s;
  }
};

// Per-kernel timing: when profiling is on (sb_profile_start), every launcher brackets its launches
// with a pair of HIP events on the launch stream; sb_profile_stop sums the elapsed times per kernel.
enum KernelId {
  K_FORWARD = 0, K_SOFTMAX, K_UPDATE_BIAS, K_UPDATE_BIAS_REG, K_MASK_SCORES,
  K_MASK_SWAP, K_MASK_FIX, K_APPLY_MASK, K_ARGMAX, K_GATHER, K_FILL, K_TRAIN_FUSED, K_MASK_ROWS, K_WEIGHT_PASS, K_COUNT
};
const char *kernel_name(int id);
struct ProfScope {
  // carried = false: the scope records an event on the stream ahead of the launches and one behind them.
  // carried = true: the launches themselves carry the events (hipExtLaunchKernelGGL takes a start and a stop
  // event and stamps them with the dispatch's own begin and end, which is what a kernel trace reports): the
  // scope records nothing, the caller passes start() to its first launch and stop() to its last.
  ProfScope(hipStream_t st, int id, bool carried = false);
  ~ProfScope();
  bool carries() const { return slot_ >= 0 && carried_; }  // the caller's launches take start() and stop()
  hipEvent_t start() const;
  hipEvent_t stop() const;
  hipStream_t st_;
  int slot_;
  bool carried_;
};
// whether the durations recorded for kernel index `id` come from events carried by the launches
bool prof_carried(int id);

void set_error(const std::string &msg);
int hip_fail(hipError_t e, const char *what, const char *file, int line);

#define SB_HIP(call)                                                 \
  do {                                                               \
    hipError_t e_ = (call);                                          \
    if (e_ != hipSuccess) return ::sb::hip_fail(e_, #call, __FILE__, __LINE__); \
  } while (0)

#define SB_REQUIRE(cond, msg)                         \
  do {                                                \
    if (!(cond)) {                                    \
      ::sb::set_error(std::string(__func__) + ": " + (msg)); \
      return -1;                                      \
    }                                                 \
  } while (0)

template <typename T>
int launch_forward(hipStream_t st, T *act, const T *x, const T *W, const T *bias, long B, long N,
                   long H, long Mc, bool softmax);
// The same followed by launch_argmax_rows on the result (pred and / or labels + correct given); layers of
// at most 32 units do both in one launch.
template <typename T>
int launch_forward_classify(hipStream_t st, T *act, const T *x, const T *W, const T *bias, long B, long N,
                            long H, long Mc, bool softmax, const T *labels, int32_t *pred,
                            unsigned long long *correct);
// The same result for a layer whose W is zero wherever wmask is 0, from the per-hypercolumn lists of
// connected rows that launch_mask_rows builds (rows: [H, cap] ascending indices, the rest -1; cap a
// multiple of 16; row_cnt: [H]); forward_rows_supported says whether the kernel takes the shape.
// x_blocked (optional): the same batch in blocks of 16 rows as launch_gather_rows_blocked lays them out,
// starting at the batch's first row; then x itself is not read.
template <typename T>
bool forward_rows_supported(const T *W, long N, long H, long Mc);
template <typename T>
int launch_forward_rows(hipStream_t st, T *act, const T *x, const T *W, const T *bias, const int *rows,
                        const int *row_cnt, long cap, long B, long N, long H, long Mc, const T *x_blocked);
// Lists of hypercolumns h0 .. h0 + count - 1 rebuilt from wmask.
int launch_mask_rows(hipStream_t st, int *rows, int *row_cnt, const uint8_t *wmask, long N, long H,
                     long cap, long h0, long count);
template <typename T>
int launch_softmax(hipStream_t st, T *act, long B, long H, long Mc);
// Fused Ci/Cj/Cij + weights (+ regularised bias when bias_mode == 1, + mask when wmask != nullptr).
// Reads the old traces from Ci/Cj and writes the new ones to Ci_next/Cj_next (distinct buffers).
// W == nullptr: the traces only.
// w_masked: the caller vouches that W is zero wherever wmask is 0; such entries may then be left alone.
// prefetch / prefetch_bytes: memory the next launches read first (the next batch), pulled into the
// memory-side cache by the tiled kernel while it waits for its Cij tiles; optional.
template <typename T>
int launch_train_fused(hipStream_t st, const T *x, const T *y, T *Cij, T *W, const T *Ci, const T *Cj,
                       T *Ci_next, T *Cj_next, const uint8_t *wmask, int bias_mode, T *bias, T *kbi,
                       long B, long N, long H, long Mc, T taupdt, T cthr, T khalf, T pmin, T taubdt,
                       bool w_masked, const void *prefetch = nullptr, size_t prefetch_bytes = 0);
// W from the traces as they are, the fused kernel's expression; wmask != nullptr: zero under zero mask bytes
// (w_masked: the caller vouches that W is zero there already, and such entries are left alone).
template <typename T>
int launch_weights_from_traces(hipStream_t st, T *W, const T *Ci, const T *Cj, const T *Cij, const uint8_t *wmask,
                               T cthr, long N, long H, long Mc, bool w_masked);
template <typename T>
int launch_add_bias(hipStream_t st, T *act, const T *bias, long B, long M);
template <typename T>
int launch_update_bias(hipStream_t st, T *bias, const T *Cj, T cthr, long M);
template <typename T>
int launch_update_bias_regularized(hipStream_t st, T *bias, T *kbi, const T *Cj, T cthr, T khalf,
                                   T pmin, T taubdt, long M);
// nom / csum: scratch of N elements each.  W == nullptr: weights recomputed from the traces.
template <typename T>
int launch_update_mask(hipStream_t st, uint8_t *wmask, const T *W, const T *Ci, const T *Cj,
                       const T *Cij, T cthr, long N, long H, long Mc, long h, long iterations, T *nom,
                       int *csum);
// The network's rewiring step: scores from the traces, the swaps, then W[:, columns of h] under the new mask
// and (rows != nullptr) the row list of h -- in the swap kernel's wake where that kernel can, else through
// launch_mask_fix_weights.
template <typename T>
int launch_rewire(hipStream_t st, uint8_t *wmask, T *W, const T *Ci, const T *Cj, const T *Cij, T cthr, long N,
                  long H, long Mc, long h, long iterations, T *nom, int *csum, int *rows, int *row_cnt,
                  long cap);
// rows != nullptr: the row list of hypercolumn h (see launch_mask_rows) is rebuilt in the same launch.
template <typename T>
int launch_mask_fix_weights(hipStream_t st, T *W, const uint8_t *wmask, const T *Ci, const T *Cj,
                            const T *Cij, T cthr, long N, long H, long Mc, long h, int *rows, int *row_cnt,
                            long cap);
template <typename T>
int launch_apply_mask(hipStream_t st, T *W, const uint8_t *wmask, long N, long H, long Mc);
template <typename T>
int launch_count_unmasked(hipStream_t st, const T *W, const uint8_t *wmask, long N, long H, long Mc,
                          unsigned long long *count);
template <typename T>
int launch_argmax_rows(hipStream_t st, const T *act, const T *labels, long B, long M, int32_t *pred,
                       unsigned long long *correct);
template <typename T>
int launch_gather_rows(hipStream_t st, T *dst, const T *src, const int64_t *idx, long rows, long cols);
// dst[(r / 16) * cols + c][r % 16] = src[idx ? idx[r] : r, c], rows of the last block beyond `rows` zero:
// ceil(rows / 16) * 16 * cols elements.  plain (optional) receives what launch_gather_rows would write.
template <typename T>
int launch_gather_rows_blocked(hipStream_t st, T *dst, T *plain, const T *src, const int64_t *idx, long rows,
                               long cols);
// `workgroups` workgroups of four wavefronts, each wavefront 8 * iters MFMAs of 2 * 16 * 16 * 4 flops.
template <typename T>
int launch_mfma_probe(hipStream_t st, T *sink, long workgroups, long iters);
// the 4x4x4 form of the fp64 MFMA: 16 * iters instructions of 2 * 4 * 4 * 4 * 4 flops per wavefront
int launch_mfma_probe_f64_4x4x4(hipStream_t st, double *sink, long workgroups, long iters);
template <typename T>
int launch_fill(hipStream_t st, T *dst, T value, size_t n);
// dst1[0 .. n1) = src1, dst2[0 .. n2) = src2 in one launch
template <typename T>
int launch_copy_pair(hipStream_t st, T *dst1, const T *src1, size_t n1, T *dst2, const T *src2, size_t n2);
int launch_fill_bytes(hipStream_t st, void *dst, int value, size_t bytes);

}  // namespace sb
