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
// one workgroup per R rows of Cij (skinny_train_rows), thread (r, j) owning one element.  The workgroup stages its
// R columns of x and all of y in LDS, `bc` batch rows at a time, with every load of a chunk in flight at
// once (a row of x contributes R consecutive elements, a row of y all M); each thread then walks the
// chunk in LDS, accumulating its x^T y element and, in batch order and without FMA contraction, the
// column sums its row's Ci and its column's Cj are made of -- the reference's order, so the traces are
// bit-exact as in the tiled kernel.  Rows past the batch are staged as zeros, which change no sum.
// bc (set by the launcher): at most kSkinnyLoads passes of either staging loop, at most kSkinnyStage
// staged elements, byte offsets of a chunk of x below 2 GiB.
// Rows of Cij per workgroup: as many as fit 256 threads, at most 32 (with fewer columns than 8 some threads
// only stage; more rows would shorten the chunks the staging loops can cover).
__host__ __device__ constexpr int skinny_train_rows(long M) { return 256 / M < 32 ? (int)(256 / M) : 32; }
constexpr int kSkinnyLoads = 16;
constexpr int kSkinnyStage = 8192;
template <typename T>
__global__ __launch_bounds__(256) void k_train_skinny(TrainArgs<T> a, int bc) {
  using Rl = Real<T>;
  __shared__ T stage[kSkinnyStage];
  const int tid = threadIdx.x;
  const int M = (int)a.M;
  const int R = skinny_train_rows(M);
  const int j = tid % M, r = tid / M;
  const long i0 = (long)blockIdx.x * R, i = i0 + r;
  const bool mine = r < R && i < a.N;  // this thread owns an element of Cij
  T *xs = stage, *ys = stage + bc * R;
  // staging roles: x by (row xb of a pass, column xr), y by (row yb, column yj)
  const int xrows = 256 / R, xb = tid / R, xr = tid % R;  // xrows * R <= 256 threads load x
  const int yrows = 256 / M, yb = tid / M, yj = tid % M;
  const bool xload = xb < xrows && i0 + xr < a.N, yload = yb < yrows;
  constexpr unsigned ES = sizeof(T);
  const T cij_old = mine ? a.Cij[i * a.M + j] : T(0);  // requested first, used last
  T dot = T(0), sx = T(0), sy = T(0);
  for (long b0 = 0; b0 < a.B; b0 += bc) {
    const long left = a.B - b0;  // rows of this chunk inside the batch: min(left, bc)
    const BufferWindow<T> xwin(a.x + b0 * a.N + i0, (left - 1) * a.N + (a.N - i0)),
        ywin(a.y + b0 * a.M, left * a.M);
    T xv[kSkinnyLoads], yv[kSkinnyLoads];
#pragma unroll
    for (int k = 0; k < kSkinnyLoads; k++) {
      const int bx = xb + k * xrows, by = yb + k * yrows;
      T one[1];
      xwin.template load_n<1>(one, xload && bx < bc ? (unsigned)(((long)bx * a.N + xr) * ES)
                                                    : BufferWindow<T>::kOutside);
      xv[k] = one[0];
      ywin.template load_n<1>(one, yload && by < bc ? (unsigned)(((long)by * a.M + yj) * ES)
                                                    : BufferWindow<T>::kOutside);
      yv[k] = one[0];
    }
    if (b0 > 0) __syncthreads();  // the previous chunk has been consumed
#pragma unroll
    for (int k = 0; k < kSkinnyLoads; k++) {
      const int bx = xb + k * xrows, by = yb + k * yrows;
      if (xb < xrows && bx < bc) xs[bx * R + xr] = xv[k];
      if (yload && by < bc) ys[by * M + yj] = yv[k];
    }
    __syncthreads();
    if (mine) {
      const int rows = left < bc ? (int)left : bc;
      for (int b = 0; b < rows; b++) {
        const T xk = xs[b * R + r], yk = ys[b * M + j];
        dot += xk * yk;
        sx = Rl::add(sx, xk);
        sy = Rl::add(sy, yk);
      }
    }
  }
  if (!mine) return;
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
  T cn = cij_old * a.omt + dot * (a.invB * a.tau);
  cn = fmax(cn, T(0));
  a.Cij[i * a.M + j] = cn;
  const T wgt = weight_from_traces<T>(cn, trace_reciprocal<T>(ci, a.cthr), trace_reciprocal<T>(cj, a.cthr),
                                      a.cthr4);
  const bool on = a.wmask == nullptr || a.wmask[i * a.H + j / (int)a.Mc] != 0;
  if (a.W) a.W[i * a.M + j] = on ? wgt : T(0);
}

}  // namespace sb
