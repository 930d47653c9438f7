// Layers with very few output units (the 10-unit classification layer): forward and training passes on
// plain vector arithmetic.  With M <= 32 output columns an MFMA tile would be mostly padding, and the
// whole problem is a few million multiply-adds whose cost is latency, not arithmetic; what matters is
// that every load is coalesced and that no thread does more than a few hundred instructions.
//
// Thread layout shared by both kernels: R = 256 / M rows of W (or Cij) per pass, thread t < R*M owns
// column j = t % M of row r = t / M, so the R*M threads of a pass read R*M consecutive elements.
#pragma once
#include "sb_kernels.hpp"

namespace sb {

// act[b, :] = softmax_per_hypercolumn(x[b, :] . W + bias)      omp.cc:70-87 + kernels_numpy.py:13-25
// One workgroup per batch row.  Partial sums over the rows r, r + R, ... are added up in the order of r
// (fixed, so the result is deterministic).
// Classification in the same launch (_cpu_base_backend.py:239-241), when pred or labels is given: the
// row's first maximal unit goes to pred[b], and *correct counts the rows whose first maximal unit is the
// labels' first maximal unit -- the result k_argmax_rows gives on the stored activations.
template <typename T>
__global__ __launch_bounds__(256) void k_forward_skinny(T *act, const T *x, const T *W, const T *bias,
                                                        long N, long M, long Mc, int softmax,
                                                        const T *labels, int32_t *pred,
                                                        unsigned long long *correct) {
  __shared__ T part[256];
  __shared__ T logit[32];
  const int tid = threadIdx.x;
  const int R = 256 / (int)M;
  const int j = tid % (int)M, r = tid / (int)M;
  const T *xrow = x + (long)blockIdx.x * N;
  T acc = T(0);
  if (r < R) {
    // pointers advance by R rows per step, so a load costs one address addition and no multiplication
    const T *xq = xrow + r, *wq = W + (long)r * M + j;
    const long wstep = (long)R * M;
    long i = r;
    for (; i + 7 * R < N; i += 8 * R) {  // 8 rows of loads in flight
      T xv[8], wv[8];
#pragma unroll
      for (int k = 0; k < 8; k++) {
        xv[k] = *xq, wv[k] = *wq;
        xq += R, wq += wstep;
      }
#pragma unroll
      for (int k = 0; k < 8; k++) acc += xv[k] * wv[k];
    }
    for (; i < N; i += R, xq += R, wq += wstep) acc += *xq * *wq;
  }
  part[tid] = acc;
  __syncthreads();
  if (tid < M) {
    T s = T(0);
    for (int k = 0; k < R; k++) s += part[k * (int)M + tid];
    logit[tid] = s + bias[tid];
  }
  __syncthreads();
  T v = T(0);
  if (tid < M) {
    v = logit[tid];
    if (softmax) {
      const int h0 = (tid / (int)Mc) * (int)Mc;  // first unit of this thread's hypercolumn
      T mx = -INFINITY;
      for (int c = 0; c < Mc; c++) mx = logit[h0 + c] > mx ? logit[h0 + c] : mx;
      T sum = T(0);
      for (int c = 0; c < Mc; c++) sum += Real<T>::exp_(logit[h0 + c] - mx);
      v = Real<T>::exp_(v - mx) / sum;
    }
    act[(long)blockIdx.x * M + tid] = v;
  }
  if (pred == nullptr && labels == nullptr) return;  // uniform
  __syncthreads();  // everybody has read the logits
  if (tid < M) logit[tid] = v;
  __syncthreads();
  if (tid == 0) {
    int best = 0;
    for (int c = 1; c < M; c++) best = logit[c] > logit[best] ? c : best;
    if (pred) pred[blockIdx.x] = best;
    if (labels) {
      const T *lab = labels + (long)blockIdx.x * M;
      int lbest = 0;
      for (int c = 1; c < M; c++) lbest = lab[c] > lab[lbest] ? c : lbest;
      if (lbest == best) atomicAdd(correct, 1ull);
    }
  }
}

// The fused training pass of k_train_fused (same arguments, same results within rounding) for M <= 32:
// one workgroup per R rows of Cij; thread (r, j) walks the batch once, accumulating its x^T y element
// and, in batch order and without FMA contraction, the column sums its row's Ci and its column's Cj
// are made of -- the reference's order, so the traces are bit-exact as in the tiled kernel.
template <typename T>
__global__ __launch_bounds__(256) void k_train_skinny(TrainArgs<T> a) {
  using Rl = Real<T>;
  const int tid = threadIdx.x;
  const int M = (int)a.M;
  const int R = 256 / M;
  const int j = tid % M, r = tid / M;
  const long i = (long)blockIdx.x * R + r;
  if (r >= R || i >= a.N) return;  // no barriers below
  T dot = T(0), sx = T(0), sy = T(0);
  const T *xp = a.x + i, *yp = a.y + j;
  // 32 batch rows of loads in flight (branch-free: past the batch the last row is re-read and counts
  // as 0), then the ordered arithmetic; the pointers advance by one row per load
  for (long b0 = 0; b0 < a.B; b0 += 32) {
    T xv[32], yv[32];
#pragma unroll
    for (int k = 0; k < 32; k++) {
      const bool live = b0 + k < a.B;  // uniform; the pointers stop at the last row of the batch
      xv[k] = *xp, yv[k] = *yp;
      xp += live && b0 + k + 1 < a.B ? a.N : 0;
      yp += live && b0 + k + 1 < a.B ? a.M : 0;
    }
#pragma unroll
    for (int k = 0; k < 32; k++) {
      const bool live = b0 + k < a.B;
      const T xk = live ? xv[k] : T(0), yk = live ? yv[k] : T(0);
      dot += xk * yk;
      sx = Rl::add(sx, xk);
      sy = Rl::add(sy, yk);
    }
  }
  const T ci = trace_next<T>(a.Ci[i], sx, a), cj = trace_next<T>(a.Cj[j], sy, a);
  if (j == 0) a.Ci_next[i] = ci;
  if (i == 0) {
    a.Cj_next[j] = cj;
    if (a.bias_mode == 1) {
      T kb = a.kbi[j];
      a.bias[j] = bias_regularized<T>(cj, kb, a.cthr, a.khalf, a.pmin, a.taubdt);
      a.kbi[j] = kb;
    }
  }
  T cn = a.Cij[i * a.M + j] * a.omt + dot * (a.invB * a.tau);
  cn = fmax(cn, T(0));
  a.Cij[i * a.M + j] = cn;
  const T wgt = weight_from_traces<T>(cn, trace_reciprocal<T>(ci, a.cthr), trace_reciprocal<T>(cj, a.cthr),
                                      a.cthr4);
  const bool on = a.wmask == nullptr || a.wmask[i * a.H + j / (int)a.Mc] != 0;
  if (a.W) a.W[i * a.M + j] = on ? wgt : T(0);
}

}  // namespace sb
