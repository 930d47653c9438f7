/*
 * sbhip.h -- C ABI of libsbhip.so, the MI355X (gfx950) backend of the BCPNN layer training and
 * inference step.
 *
 * Conventions
 *   - plain C types only; every function returns 0 on success or a negative sb_status, never
 *     exits the process (the reference's CUDA path calls exit() on error,
 *     BCPNN/backend/full_cuda_backend/helpers_cuda.h:7-27); sb_last_error() gives the message.
 *   - "d_" pointers are device (HBM) pointers, "h_" pointers are host pointers.
 *   - all matrices are dense row-major: x[B,N], y[B,M], W[N,M], Cij[N,M], wmask[N,H] (uint8).
 *     N = in_features, H = hypercolumns, Mc = minicolumns, M = H*Mc, B = batch rows.
 *   - every launch goes to one library-owned stream, in call order; calls return without waiting
 *     for the GPU unless stated.  A handle must not be used from two threads at once.
 *   - the _f32 / _f64 suffix is the element type of every real-valued array of that call.
 *
 * The per-kernel entry points carry the names of the reference's kernel module
 * (BCPNN/backend/_kernels/kernels_openmp_internal.cc:460-478); the sb_net_* entry points are what a
 * pybind11 backend object of the shape of PyNetwork<REAL>
 * (BCPNN/backend/full_cuda_backend/backend_full_cuda_internals.cu:648-781) binds.
 */
#ifndef SBHIP_H
#define SBHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum sb_status {
  SB_OK = 0,
  SB_ERR_INVALID = -1,   /* bad argument: null pointer, non-positive size, h >= H, ... */
  SB_ERR_HIP = -2,       /* a HIP runtime call failed */
  SB_ERR_STATE = -3,     /* call order: no dataset, unknown layer, not initialised */
  SB_ERR_UNSUPPORTED = -4
} sb_status;

typedef enum sb_dtype { SB_F32 = 0, SB_F64 = 1 } sb_dtype;

/* ---- library ---------------------------------------------------------------------------------
 * sb_init replaces the module-level initialize() of the reference's GPU backend
 * (backend_full_cuda_internals.cu:757-762): selects the device and creates the stream. */
int sb_init(int device);
int sb_shutdown(void);
const char *sb_last_error(void);
int sb_abi_version(void);
/* Blocks until everything enqueued so far has finished. */
int sb_sync(void);
/* The library's stream as a hipStream_t, for callers that time or order work with HIP events. */
void *sb_stream(void);

/* Number of allocating runtime calls (device and pinned host memory, events) the library has made so far
 * in this process: a call that promises to allocate nothing leaves it unchanged.  No counterpart in the
 * reference. */
long sb_allocation_calls(void);

/* ---- device memory for callers that have no HIP runtime of their own (ctypes tests, bench) --- */
int sb_malloc(void **d_ptr, size_t bytes);
int sb_free(void *d_ptr);
int sb_memcpy_h2d(void *d_dst, const void *h_src, size_t bytes); /* synchronous */
int sb_memcpy_d2h(void *h_dst, const void *d_src, size_t bytes); /* synchronous */
int sb_memcpy_d2d(void *d_dst, const void *d_src, size_t bytes); /* stream-ordered */
int sb_fill_bytes(void *d_dst, int value, size_t bytes);         /* stream-ordered fill kernel */

/* ---- per-kernel entry points (device pointers) ------------------------------------------------ */

/* act[B,M] = x[B,N] . W[N,M] + bias[M]   (act is overwritten)
 * replaces update_state_float32/64 -> matmul_add_bias, kernels_openmp_internal.cc:70-87,342-358 */
int sb_update_state_f32(float *d_act, const float *d_x, const float *d_W, const float *d_bias,
                        long B, long N, long M);
int sb_update_state_f64(double *d_act, const double *d_x, const double *d_W, const double *d_bias,
                        long B, long N, long M);

/* in place: softmax over the Mc minicolumns of each of the H hypercolumns of each row
 * replaces softmax_minicolumns, kernels_numpy.py:13-25 (bound by cpu_backend.py:10,24) */
int sb_softmax_minicolumns_f32(float *d_act, long B, long H, long Mc);
int sb_softmax_minicolumns_f64(double *d_act, long B, long H, long Mc);

/* update_state followed by softmax_minicolumns in one launch (layer.compute_activation,
 * _cpu_base_backend.py:44-51,126-133) */
int sb_compute_activation_f32(float *d_act, const float *d_x, const float *d_W,
                              const float *d_bias, long B, long N, long H, long Mc);
int sb_compute_activation_f64(double *d_act, const double *d_x, const double *d_W,
                              const double *d_bias, long B, long N, long H, long Mc);

/* compute_activation for a masked layer: W must be zero wherever wmask is 0 (the state apply_mask,
 * kernels_openmp_internal.cc:322-335, leaves behind), and the reduction then runs over the connected
 * rows only.  sb_mask_rows builds what it needs from wmask[N,H]: d_rows[H,cap] = ascending indices
 * of the set bytes of each column, then -1 up to cap (cap: a multiple of 16, at least
 * the largest column count rounded up), d_row_cnt[H] = the column counts.  Same result as
 * sb_compute_activation on such a W, up to the order of the sum.  Needs Mc and H*Mc divisible by 4
 * (f32) or 2 (f64), Mc <= 256 (f32) or 224 (f64), 16-byte aligned W. */
int sb_mask_rows(int *d_rows, int *d_row_cnt, const unsigned char *d_wmask, long N, long H, long cap);
int sb_compute_activation_rows_f32(float *d_act, const float *d_x, const float *d_W,
                                   const float *d_bias, const int *d_rows, const int *d_row_cnt,
                                   long cap, long B, long N, long H, long Mc, const float *d_x_blocked);
int sb_compute_activation_rows_f64(double *d_act, const double *d_x, const double *d_W,
                                   const double *d_bias, const int *d_rows, const int *d_row_cnt,
                                   long cap, long B, long N, long H, long Mc, const double *d_x_blocked);
/* d_x_blocked (optional, may be NULL): the same batch in blocks of 16 rows, as sb_rows_in_blocks lays it
 * out: d_dst[(r / 16) * cols + c][r % 16] = d_src[r, c], ceil(rows / 16) * 16 * cols elements, rows past
 * the last one zero.  The kernel then reads a picked input column of 16 batch rows as one 64-byte run
 * instead of 16 scattered elements, and d_x itself is not read. */
int sb_rows_in_blocks_f32(float *d_dst, const float *d_src, long rows, long cols);
int sb_rows_in_blocks_f64(double *d_dst, const double *d_src, long rows, long cols);

/* The two halves of update_weights as the reference's cuda kernel set has them
 * (BCPNN/backend/_kernels/kernels_cuda.py:40-59), and its separate bias step (:18-26):
 *   sb_update_counters        Ci, Cj, Cij moving averages only (kernels_openmp_internal.cc:89-190)
 *   sb_weights_from_counters  W from the traces as they are (:192-199), unmasked
 *   sb_add_bias               act[b, j] += bias[j] */
int sb_update_counters_f32(float *d_Ci, float *d_Cj, float *d_Cij, const float *d_a_i, const float *d_a_o,
                           float taupdt, long B, long N, long M);
int sb_update_counters_f64(double *d_Ci, double *d_Cj, double *d_Cij, const double *d_a_i,
                           const double *d_a_o, double taupdt, long B, long N, long M);
int sb_weights_from_counters_f32(float *d_W, const float *d_Ci, const float *d_Cj, const float *d_Cij,
                                 float cthr, long N, long M);
int sb_weights_from_counters_f64(double *d_W, const double *d_Ci, const double *d_Cj, const double *d_Cij,
                                 double cthr, long N, long M);
/* sb_weights_from_counters followed by sb_apply_mask in one pass over Cij and W (the weight recompute fused
 * with the mask apply: kernels_openmp_internal.cc:192-199 then :322-335): W[i, j] is the weight where
 * wmask[i, j / Mc] is set and 0 elsewhere; Cij under zero mask bytes is not read. */
int sb_weights_masked_from_counters_f32(float *d_W, const float *d_Ci, const float *d_Cj, const float *d_Cij,
                                        const uint8_t *d_wmask, float cthr, long N, long H, long Mc);
int sb_weights_masked_from_counters_f64(double *d_W, const double *d_Ci, const double *d_Cj, const double *d_Cij,
                                        const uint8_t *d_wmask, double cthr, long N, long H, long Mc);
int sb_add_bias_f32(float *d_act, const float *d_bias, long B, long M);
int sb_add_bias_f64(double *d_act, const double *d_bias, long B, long M);

/* Ci, Cj, Cij moving averages (clamped at 0) and W = log(max(Cij,cthr^4)/(Ci*Cj)) with rows
 * Ci<cthr and columns Cj<cthr zeroed; all in place; W is the unmasked weight.
 * replaces update_weights_float32/64 -> vectorized_updateWeights,
 * kernels_openmp_internal.cc:89-205,361-383 */
int sb_update_weights_f32(float *d_Ci, float *d_Cj, float *d_Cij, const float *d_a_i,
                          const float *d_a_o, float taupdt, float *d_W, float cthr, long B, long N,
                          long M);
int sb_update_weights_f64(double *d_Ci, double *d_Cj, double *d_Cij, const double *d_a_i,
                          const double *d_a_o, double taupdt, double *d_W, double cthr, long B,
                          long N, long M);

/* sb_update_weights_f32 for callers that cannot call hipMalloc (tight serving loops, harnesses that
 * forbid allocation; the launches go to the library's own stream, so this is not something a caller's
 * stream capture could record).  No counterpart in the reference.  Same arguments
 * and results as sb_update_weights_f32; the intermediate new Ci / Cj live in a static device array of
 * SB_NOALLOC_MAX_UNITS floats (1 MiB, held by every GPU the library runs on until the process ends)
 * instead of a buffer the library grows on demand, so the call allocates and frees nothing.  Returns
 * SB_ERR_UNSUPPORTED when N + M > SB_NOALLOC_MAX_UNITS, SB_ERR_STATE between sb_profile_start and
 * sb_profile_stop (event brackets allocate).  Every call of a process on a GPU shares the one array,
 * which keeps the last call's contents (the kernel overwrites what it reads back, nothing needs
 * clearing): two calls that overlapped on a GPU would race.  The library's single stream orders them;
 * as with every entry point, do not call from two threads at once. */
#define SB_NOALLOC_MAX_UNITS 262144
int sb_update_weights_noalloc_f32(float *d_Ci, float *d_Cj, float *d_Cij, const float *d_a_i,
                                  const float *d_a_o, float taupdt, float *d_W, float cthr, long B,
                                  long N, long M);

/* replaces update_bias_float32/64, kernels_openmp_internal.cc:207-220,386-396 */
int sb_update_bias_f32(float *d_bias, const float *d_Cj, float cthr, long M);
int sb_update_bias_f64(double *d_bias, const double *d_Cj, double cthr, long M);

/* replaces update_bias_regularized_float32/64, kernels_openmp_internal.cc:222-246,399-415 */
int sb_update_bias_regularized_f32(float *d_bias, float *d_kbi, const float *d_Cj, float cthr,
                                   float khalf, float pmin, float taubdt, long M);
int sb_update_bias_regularized_f64(double *d_bias, double *d_kbi, const double *d_Cj, double cthr,
                                   double khalf, double pmin, double taubdt, long M);

/* Structural-plasticity rewiring of hypercolumn h: up to `iterations` greedy swaps between the
 * best-scoring silent row and the worst-scoring active row of wmask[:, h] (ties: highest row index).
 * replaces update_mask_float32/64, kernels_openmp_internal.cc:248-320,418-441 */
int sb_update_mask_f32(uint8_t *d_wmask, const float *d_W, const float *d_Ci, const float *d_Cj,
                       const float *d_Cij, float cthr, long N, long H, long Mc, long h,
                       long iterations);
int sb_update_mask_f64(uint8_t *d_wmask, const double *d_W, const double *d_Ci, const double *d_Cj,
                       const double *d_Cij, double cthr, long N, long H, long Mc, long h,
                       long iterations);

/* W[i,j] = 0 where wmask[i, j / Mc] == 0
 * replaces apply_mask_float32/64, kernels_openmp_internal.cc:322-335,444-458 */
int sb_apply_mask_f32(float *d_W, const uint8_t *d_wmask, long N, long H, long Mc);
int sb_apply_mask_f64(double *d_W, const uint8_t *d_wmask, long N, long H, long Mc);

/* d_pred[b] = index of the first maximum of act[b, :]  (np.argmax, _cpu_base_backend.py:239) */
int sb_argmax_rows_f32(const float *d_act, long B, long M, int32_t *d_pred);
int sb_argmax_rows_f64(const double *d_act, long B, long M, int32_t *d_pred);

/* One structural-plasticity layer training step on device-resident state, in the order of
 * StructuralPlasticityLayer.train_step (cpu_backend.py:29-52): traces + weights, regularised bias,
 * [mask rewiring of hypercolumn h when h >= 0, 16 iterations], mask apply.  d_W holds the MASKED
 * weights on return.  d_x is the layer input, d_y its activation for the same batch. */
int sb_plastic_train_step_f32(float *d_W, float *d_bias, float *d_Ci, float *d_Cj, float *d_Cij,
                              float *d_kbi, uint8_t *d_wmask, const float *d_x, const float *d_y,
                              long B, long N, long H, long Mc, float taupdt, float khalf,
                              float pmin, float taubdt, long h);
int sb_plastic_train_step_f64(double *d_W, double *d_bias, double *d_Ci, double *d_Cj,
                              double *d_Cij, double *d_kbi, uint8_t *d_wmask, const double *d_x,
                              const double *d_y, long B, long N, long H, long Mc, double taupdt,
                              double khalf, double pmin, double taubdt, long h);

/* ---- network object ---------------------------------------------------------------------------
 * Device-resident counterpart of Network<REAL>/PyNetwork<REAL>
 * (backend_full_cuda_internals.cu:481-644,648-754) with the cpu backend's semantics
 * (_cpu_base_backend.py:175-314, cpu_backend.py:7-52). */
typedef struct sb_net sb_net;

int sb_net_create(sb_net **net, int dtype /* sb_dtype */);
int sb_net_destroy(sb_net *net);

/* PyNetwork::add_dense_layer (backend_full_cuda_internals.cu:653-665): counters start at the three
 * initial values; weights and bias start at zero and the mask of a plastic layer at all ones until
 * sb_net_randomize_layer or sb_net_set_layer_state gives them values (a layer left at zero weights cannot
 * learn: every softmax stays uniform).  Returns the layer index (>= 0) or a negative sb_status. */
int sb_net_add_dense_layer(sb_net *net, long n_inputs, long hypercolumns, long minicolumns,
                           double taupdt, double initial_Ci, double initial_Cj,
                           double initial_Cij);
/* PyNetwork::add_plastic_layer (backend_full_cuda_internals.cu:667-683); note pmin before khalf. */
int sb_net_add_plastic_layer(sb_net *net, long n_inputs, long hypercolumns, long minicolumns,
                             double taupdt, double pmin, double khalf, double taubdt,
                             double initial_Ci, double initial_Cj, double initial_Cij);

/* The initial state the reference's GPU backend object draws when a layer is constructed
 * (backend_full_cuda_internals.cu:151-155: weights ~ N(0, 0.1), bias ~ 0.1 U(0, 1);
 * helpers_training.cu:10-32: each mask byte of a plastic layer set with probability 0.1 -- `density`
 * here), from a 64-bit Mersenne twister seeded with `seed`: the same seed gives the same state.  Drawn on
 * the host and uploaded; synchronous.  sb_net_set_layer_state afterwards overrides any of it. */
int sb_net_randomize_layer(sb_net *net, int layer, uint64_t seed, double density);

/* State arrays of a layer, by name: "weights" [N,M], "bias" [M], "Ci" [N], "Cj" [M], "Cij" [N,M],
 * "kbi" [M] (plastic layers) in the network dtype, and "wmask" [N,H] uint8 (plastic layers).
 * The reference keeps these as numpy attributes of the layer (_cpu_base_backend.py:31-42,107-124);
 * `bytes` must equal the array's size.  Both calls are synchronous. */
int sb_net_set_layer_state(sb_net *net, int layer, const char *name, const void *h_src,
                           size_t bytes);
int sb_net_get_layer_state(sb_net *net, int layer, const char *name, void *h_dst, size_t bytes);

/* PyNetwork::initiate_training (backend_full_cuda_internals.cu:685-709): copies the training set
 * (network dtype, images [n_samples, n_features], one-hot labels [n_samples, n_classes]) to HBM.
 * h_labels may be NULL when only non-final layers are trained. */
int sb_net_set_training_data(sb_net *net, const void *h_images, const void *h_labels,
                             long n_samples, long n_features, long n_classes);
/* PyNetwork::training_done (backend_full_cuda_internals.cu:715-722): releases the training set. */
int sb_net_training_done(sb_net *net);

/* One epoch of Network._train_layer (_cpu_base_backend.py:254-314) for `layer`:
 *   h_sample_perm[n_samples]  the epoch's sample order (int64), batches are consecutive slices of
 *                             maximal_batch_size rows, the last one short;
 *   h_hc_perm[H]              the epoch's hypercolumn order (int64) for the rewiring schedule
 *                             (:297-302), used when epoch_index > 0; may be NULL for the last layer;
 * the last layer trains on the labels, any other on its own activation; ends with train_finalize.
 * When n_batches / (H + 1) is zero the reference divides by zero; here no rewiring happens.
 * While the last layer trains, the layers below it do not change: their activations of the training set
 * are computed in its first epoch and kept (two copies of [n_samples, its input width], as long as
 * they stay below 16 GiB and half of the free device memory) until a lower layer trains, state is written or the training set is replaced.
 * Asynchronous: returns once the epoch is enqueued. */
int sb_net_train_epoch(sb_net *net, int layer, long maximal_batch_size,
                       const int64_t *h_sample_perm, const int64_t *h_hc_perm, long epoch_index);

/* Upper bound, in bytes (both copies together), of the cache of frozen layers' activations that
 * sb_net_train_epoch keeps while the last layer trains; 16 GiB unless set.  0 switches the cache off: every
 * step then runs the forward passes of the layers below, as the reference does
 * (_cpu_base_backend.py:279-295), with identical results.  A cache already held that exceeds the new bound
 * is dropped. */
int sb_net_set_frozen_cache_limit(sb_net *net, size_t bytes);

/* A contiguous range of an epoch's batches [first_batch, first_batch + n_batches): sb_net_train_epoch
 * is the whole range with finalize = 1.  The sample order is applied when first_batch == 0 (it may be
 * NULL otherwise); later ranges continue the same epoch.  For callers that interleave their own work
 * (progress reporting as in _cpu_base_backend.py:270-312, timing) with an epoch. */
int sb_net_train_batches(sb_net *net, int layer, long maximal_batch_size,
                         const int64_t *h_sample_perm, const int64_t *h_hc_perm, long epoch_index,
                         long first_batch, long n_batches, int finalize);

/* Network.evaluate (_cpu_base_backend.py:205-245): forward through every layer, count rows whose
 * argmax equals the label's argmax.  Synchronous.  h_pred (may be NULL) receives the predicted
 * class per row.  The host arrays go up in pieces through pinned staging buffers while earlier pieces are
 * computed; the device buffers of a chunk of the set (at most about 2 x 256 MiB of images, plus labels and
 * predictions) are kept with the network for the next call and released by sb_net_destroy. */
int sb_net_evaluate(sb_net *net, const void *h_images, const void *h_labels, long n_samples,
                    long n_features, long n_classes, long maximal_batch_size, int64_t *correct,
                    int64_t *total, int32_t *h_pred);

/* Predicted class (first maximal activation of the last layer, np.argmax) per row of host images;
 * the labels-free half of Network.evaluate (_cpu_base_backend.py:235-239).  Synchronous. */
int sb_net_predict(sb_net *net, const void *h_images, long n_samples, long n_features,
                   long maximal_batch_size, int32_t *h_pred);

/* Forward of rows [0, n_rows) of host images through layers 0..last_layer; the activation of
 * last_layer [n_rows, M_last] is copied to h_act.  Synchronous. */
int sb_net_forward(sb_net *net, const void *h_images, long n_rows, long n_features, int last_layer,
                   long maximal_batch_size, void *h_act);

/* The layer-level calls of the DSL on one layer of the network, on host arrays in the network dtype
 * (_cpu_base_backend.py:44-51,126-133 compute_activation; cpu_backend.py:13-18,29-52 train_step and
 * train_finalize).  Synchronous.
 *   sb_net_layer_activation      h_act[n_rows, M] = softmax_hc(h_inputs[n_rows, N] . W + bias) of `layer`
 *   sb_net_layer_train_step      one training step of `layer` on inputs [n_rows, N] and outputs [n_rows, M]
 *                                (its own activation, or the labels for the last layer); hypercolumn >= 0
 *                                also rewires that hypercolumn (structural-plasticity layers), -1: none
 *   sb_net_layer_train_finalize  dense layers: bias from Cj; structural-plasticity layers: nothing */
int sb_net_layer_activation(sb_net *net, int layer, const void *h_inputs, long n_rows, void *h_act);
int sb_net_layer_train_step(sb_net *net, int layer, const void *h_inputs, const void *h_outputs, long n_rows,
                            long hypercolumn);
int sb_net_layer_train_finalize(sb_net *net, int layer);

/* ---- per-kernel timing -------------------------------------------------------------------------
 * Between sb_profile_start and sb_profile_stop every kernel launch of the library is bracketed by HIP
 * events on the library's stream; afterwards sb_profile_get returns, per kernel index in
 * [0, sb_profile_kernels()), the summed elapsed time and the number of launches.  The reference has no
 * counterpart (it times whole runs with time.time(), train.py:181-193).  The sums are raw bracket times:
 * a bracket adds a few microseconds of its own to a short kernel (compare the bracketed sum of a run
 * with its unbracketed wall time to calibrate).  The fused training launch is the exception: its events ride on
 * the launch itself (sb_profile_kernel_carried), except under rocprofv3, where they would read long and the
 * launch is bracketed like the others. */
int sb_profile_start(void);
int sb_profile_stop(void);
int sb_profile_kernels(void);
/* Elapsed time of an empty event bracket as measured by the last sb_profile_start: an upper bound of
 * what a bracket adds to a launch. */
double sb_profile_bracket_overhead_us(void);
const char *sb_profile_kernel_name(int kernel);
/* 1 when the launches of that kernel carry their events themselves (stamped with the dispatch's own begin and
 * end, as a kernel trace reports them: nothing to subtract), 0 when the events are records on the stream
 * around the launches (which add what sb_profile_bracket_overhead_us bounds). */
int sb_profile_kernel_carried(int kernel);
int sb_profile_get(int kernel, double *total_ms, long *launches);

/* Matrix-core probe for the achievable-peak record of bench.py: `workgroups` workgroups of four wavefronts
 * that issue nothing but 16x16x4 MFMAs of the given element type (8 * iters each), or, with
 * SB_PROBE_F64_4X4X4, the 4x4x4 form of the fp64 MFMA (16 * iters each); *flops receives the launch's
 * floating-point operations.  Stream-ordered; time it between sb_sync calls.  No counterpart in the
 * reference. */
#define SB_PROBE_F64_4X4X4 2
int sb_probe_mfma(int dtype /* sb_dtype or SB_PROBE_F64_4X4X4 */, long workgroups, long iters, double *flops);

#ifdef __cplusplus
}
#endif
#endif /* SBHIP_H */
