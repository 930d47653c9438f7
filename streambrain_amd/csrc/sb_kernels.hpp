// gfx950 kernels of the BCPNN layer step.  One wavefront = 64 lanes; lane = 16*q + p throughout.
//
// Reference semantics restated by each kernel are cited as file:line of the reference checkout
// ("omp.cc" = BCPNN/backend/_kernels/kernels_openmp_internal.cc).
#pragma once
#include "sb_common.hpp"

namespace sb {

// Softmax over each (row, hypercolumn) group of Mc values, in place; one wavefront per group.
// kernels_numpy.py:13-25
template <typename T>
__global__ __launch_bounds__(256) void k_softmax(T *act, long groups, long Mc) {
  const int lane = threadIdx.x & 63;
  const long g = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (g >= groups) return;
  T *v = act + g * Mc;
  T mx = -INFINITY;
  for (long c = lane; c < Mc; c += 64) mx = v[c] > mx ? v[c] : mx;
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    const T other = __shfl_xor(mx, o);
    mx = other > mx ? other : mx;
  }
  T sum = T(0);
  for (long c = lane; c < Mc; c += 64) {
    const T e = Real<T>::exp_(v[c] - mx);
    v[c] = e;
    sum += e;
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) sum += __shfl_xor(sum, o);
  for (long c = lane; c < Mc; c += 64) v[c] = v[c] / sum;
}

// update_bias_regularized for one unit (omp.cc:222-246); kbi is updated in place.
template <typename T>
__device__ __forceinline__ T bias_regularized(T pj, T &kbi, T cthr, T khalf, T pmin, T taubdt) {
  using R = Real<T>;
  const T p4 = R::div(pmin, T(4));
  const T k = R::mul(khalf - T(1), R::mul(p4, p4));
  const T d = pj - p4;
  T kb = R::add(T(1), R::div(k, R::mul(d, d)));
  if (pj < p4 || kb < khalf) kb = khalf;
  kbi = R::add(R::mul(T(1) - taubdt, kbi), R::mul(taubdt, kb));
  return (pj < cthr) ? R::mul(kbi, R::log_(R::mul(T(2), cthr))) : R::mul(kbi, R::log_(pj));
}

// omp.cc:207-220
template <typename T>
__global__ __launch_bounds__(256) void k_update_bias(T *bias, const T *Cj, T cthr, long M) {
  const long j = (long)blockIdx.x * 256 + threadIdx.x;
  if (j >= M) return;
  const T c = Cj[j];
  bias[j] = (c < cthr) ? Real<T>::log_(Real<T>::mul(T(2), cthr)) : Real<T>::log_(c);
}

// omp.cc:222-246
template <typename T>
__global__ __launch_bounds__(256) void k_update_bias_regularized(T *bias, T *kbi, const T *Cj, T cthr,
                                                                 T khalf, T pmin, T taubdt, long M) {
  const long j = (long)blockIdx.x * 256 + threadIdx.x;
  if (j >= M) return;
  T kb = kbi[j];
  bias[j] = bias_regularized<T>(Cj[j], kb, cthr, khalf, pmin, taubdt);
  kbi[j] = kb;
}

// act[b, j] += bias[j]   (the separate bias step of the reference's cuda kernel set, kernels_cuda.py:18-26)
template <typename T>
__global__ __launch_bounds__(256) void k_add_bias(T *act, const T *bias, long B, long M) {
  const long total = B * M;
  const long stride = (long)gridDim.x * 256;
  for (long e = (long)blockIdx.x * 256 + threadIdx.x; e < total; e += stride) act[e] += bias[e % M];
}

// W[i, j] from the traces as they are (omp.cc:192-199 on its own; kernels_cuda.py:51-59 has it as a
// separate step): the same expression as the fused training kernel.
template <typename T>
__global__ __launch_bounds__(256) void k_weights_from_traces(T *W, const T *Ci, const T *Cj, const T *Cij,
                                                             T cthr, T cthr4, long N, long M) {
  for (long i = blockIdx.x; i < N; i += gridDim.x) {
    const T rci = trace_reciprocal<T>(Ci[i], cthr);
    for (long j = threadIdx.x; j < M; j += 256)
      W[i * M + j] = weight_from_traces<T>(Cij[i * M + j], rci, trace_reciprocal<T>(Cj[j], cthr), cthr4);
  }
}

// The weight pass on its own, with or without the mask (omp.cc:192-199 followed by apply_mask, :322-335):
//   W[i, j] = wmask[i, j / Mc] ? log(max(Cij, cthr^4) / (Ci Cj)) : 0      (0 as well where Ci or Cj < cthr)
// for rows that are whole 16-byte vectors (M, and with a mask Mc, multiples of VW).  Bound by HBM: it reads Cij
// and writes W once, 2 s N M bytes, plus the N H mask bytes.  A thread owns VW consecutive columns (their
// column reciprocals computed once) of kRowsPerTurn rows: all its loads are in flight before the first is used.
// Cij and W are reached through bounds-checked windows over the rows of a turn (rows past the matrix read
// zero and store nothing), so the loop has no guards; under a zero mask byte the Cij vector is not read at all
// (an offset outside the window costs no memory access), and with `w_masked` -- the caller vouches that W
// holds zero there already -- not written either.  Stores write through (agent scope): with the default
// policy they sit in the L2s until the kernel ends and are written back then, which is serial time.
// Grid: x over blocks of 256 VW columns, y over row groups.
constexpr int kRowsPerTurn = 8;
template <typename T, bool MASKED>
__global__ __launch_bounds__(256) void k_weight_pass(T *W, const T *Ci, const T *Cj, const T *Cij,
                                                     const uint8_t *wmask, T cthr, T cthr4, long N, long M, long H,
                                                     FastDiv by_Mc, int w_masked) {
  constexpr int VW = Real<T>::VW;
  constexpr unsigned ES = sizeof(T), kOutside = BufferWindow<T>::kOutside;
  using vec_t = typename Real<T>::vec_t;
  const long j = ((long)blockIdx.x * 256 + threadIdx.x) * VW;
  const bool col_ok = j < M;
  T rcj[VW];
  {
    const BufferWindow<T> jwin(Cj, M);
    T cj[VW];
    jwin.load_vec(cj, col_ok ? (unsigned)j * ES : kOutside, 0);
#pragma unroll
    for (int e = 0; e < VW; e++) rcj[e] = trace_reciprocal<T>(cj[e], cthr);
  }
  const unsigned hc = MASKED && col_ok ? by_Mc.div((uint32_t)j) : 0u;
  const unsigned row_bytes = (unsigned)M * ES;  // kRowsPerTurn rows stay below 2 GiB (launcher)
  for (long i0 = (long)blockIdx.y * kRowsPerTurn; i0 < N; i0 += (long)gridDim.y * kRowsPerTurn) {
    const long rows = N - i0 < kRowsPerTurn ? N - i0 : kRowsPerTurn;
    const unsigned turn_bytes = (unsigned)rows * row_bytes;
    const BufferWindow<T> cwin(uniform_pointer(Cij + i0 * M), typename BufferWindow<T>::Bytes{turn_bytes}),
        wwin(uniform_pointer(W + i0 * M), typename BufferWindow<T>::Bytes{turn_bytes});
    uint32_t on[kRowsPerTurn];
    if constexpr (MASKED) {
      const ByteWindow mwin(uniform_pointer(wmask + i0 * H), rows * H);
#pragma unroll
      for (int r = 0; r < kRowsPerTurn; r++) on[r] = mwin.load((unsigned)(r * H) + hc, 0);
    }
    T c[kRowsPerTurn][VW], ci[kRowsPerTurn];
#pragma unroll
    for (int r = 0; r < kRowsPerTurn; r++) {
      const bool connected = !MASKED || on[r] != 0;
      cwin.load_vec(c[r], col_ok && connected ? r * row_bytes + (unsigned)j * ES : kOutside, 0);
      ci[r] = Ci[i0 + r < N ? i0 + r : N - 1];
    }
#pragma unroll
    for (int r = 0; r < kRowsPerTurn; r++) {
      const bool connected = !MASKED || on[r] != 0;
      const T ri = trace_reciprocal<T>(ci[r], cthr);
      T w[VW];
#pragma unroll
      for (int e = 0; e < VW; e++) w[e] = connected ? weight_from_traces<T>(c[r][e], ri, rcj[e], cthr4) : T(0);
      const bool skip = MASKED && w_masked && !connected;
      wwin.store_vec(w, col_ok && !skip ? r * row_bytes + (unsigned)j * ES : kOutside, 0);
    }
  }
}

// omp.cc:322-335.  A row of W per workgroup and turn; the hypercolumn of a column is a multiplication by a
// constant the host prepares (M < 2^31).
template <typename T>
__global__ __launch_bounds__(256) void k_apply_mask(T *W, const uint8_t *wmask, long N, long M, long H,
                                                    FastDiv by_Mc) {
  for (long i = blockIdx.x; i < N; i += gridDim.x) {
    T *row = W + i * M;
    const uint8_t *mrow = wmask + i * H;
    for (unsigned j = threadIdx.x; j < (unsigned)M; j += 256)
      if (mrow[by_Mc.div(j)] == 0) row[j] = T(0);
  }
}

// The same for M and Mc multiples of VW and a 16-byte aligned W: a thread owns VW consecutive columns (one
// hypercolumn) and stores 16-byte zero vectors; nothing of W is read.  Grid as k_weight_pass.
template <typename T>
__global__ __launch_bounds__(256) void k_apply_mask_vec(T *W, const uint8_t *wmask, long N, long M, long H,
                                                        FastDiv by_Mc) {
  constexpr int VW = Real<T>::VW;
  using vec_t = typename Real<T>::vec_t;
  const long j = ((long)blockIdx.x * 256 + threadIdx.x) * VW;
  if (j >= M) return;
  const uint8_t *mcol = wmask + by_Mc.div((uint32_t)j);
  vec_t zero;
#pragma unroll
  for (int e = 0; e < VW; e++) zero[e] = T(0);
  for (long i0 = (long)blockIdx.y * kRowsPerTurn; i0 < N; i0 += (long)gridDim.y * kRowsPerTurn) {
    uint8_t m[kRowsPerTurn];
#pragma unroll
    for (int r = 0; r < kRowsPerTurn; r++) m[r] = mcol[(i0 + r < N ? i0 + r : N - 1) * H];
#pragma unroll
    for (int r = 0; r < kRowsPerTurn; r++)
      if (i0 + r < N && m[r] == 0) *reinterpret_cast<vec_t *>(W + (i0 + r) * M + j) = zero;
  }
}

// Counts the entries of W that are not +0 / -0 although their mask byte is 0 (0 means: W is in the state
// apply_mask leaves behind).  NaN counts as non-zero.
template <typename T>
__global__ __launch_bounds__(256) void k_count_unmasked(const T *W, const uint8_t *wmask, long N, long M,
                                                        long H, long Mc, unsigned long long *count) {
  unsigned long long mine = 0;
  for (long i = blockIdx.x; i < N; i += gridDim.x) {  // a row of W per workgroup and turn
    const T *row = W + i * M;
    const uint8_t *mrow = wmask + i * H;
    for (unsigned j = threadIdx.x; j < (unsigned)M; j += 256)  // M < 2^31: 32-bit division
      mine += (mrow[j / (unsigned)Mc] == 0 && !(row[j] == T(0))) ? 1 : 0;
  }
  if (__syncthreads_or(mine != 0) && mine != 0) atomicAdd(count, mine);
}

// =====================================================================================================
// Structural-plasticity rewiring of one hypercolumn                      omp.cc:248-320
// Step 1 (k_mask_scores): per input row, the score nominator over the Mc columns of hypercolumn h and
//   the number of hypercolumns the row is connected to.  One wavefront per row.  When W is nullptr the
//   (unmasked) weight is recomputed from the traces with the trace/weight kernel's own formula.
// Step 2 (k_mask_swap): one workgroup repeats up to `iterations` times: best silent row (max score,
//   highest index among equals), worst active row (min score, highest index among equals), swap unless
//   vmax0 < vmin1.  The quotient nominator / (1 + csum) is formed in double and narrowed, as the
//   reference's expression does.  A NaN score behaves as in a sequential scan with >= / <=: it is
//   picked only when it belongs to the first candidate row.
// Step 3 (k_mask_fix_weights): rewrites W[:, hypercolumn h] under the new mask (network path only,
//   where W is kept masked).
// Step 4: see mask_rows_block below.
// =====================================================================================================
template <typename T>
struct MaskArgs {
  uint8_t *wmask;
  const T *W;  // may be nullptr
  const T *Ci, *Cj, *Cij;
  T cthr, cthr4;
  long N, M, H, Mc, h, iterations;
  T *nom;     // [N] scratch
  int *csum;  // [N] scratch
  // Network path (k_mask_swap_reg only): after the swaps the same workgroup rewrites W[i, columns of h] of
  // the rows that changed sides under the new mask (steps 3) and, with a row list, rebuilds the list of
  // hypercolumn h (step 4).  W_fix == nullptr: neither.
  T *W_fix;
  int *rows, *row_cnt;
  long cap;
};
constexpr int kMaxChangedRows = 64;  // rows that change sides in one merged launch: two per iteration

// One wavefront per input row.  The score nominator is the reference's own expression, operation by operation
// (omp.cc:257-277): every product, difference, quotient and sum rounded once, the logarithms accurate to the
// last bit or so (evaluated in double and narrowed for floats), and the Mc terms of a row added in ascending
// column order starting from zero -- so that two builds that start from the same traces pick the same rows.
// The lanes evaluate 64 terms at a time; the sum then walks them in order (lane by lane through scalar
// registers), which every lane does for itself.  Without a W array (the network path, where W is kept masked)
// the weight is recomputed as the reference's weight pass forms it (omp.cc:192-199): log(max(Cij, cthr^4) /
// (Ci Cj)) with the product and the quotient rounded like there.
template <typename T>
__device__ __forceinline__ T accurate_log(T x) {
  if constexpr (sizeof(T) == 4) return (T)log((double)x);
  else return log(x);
}
template <typename T>
__global__ __launch_bounds__(256) void k_mask_scores(MaskArgs<T> a) {
  using R = Real<T>;
  const int lane = threadIdx.x & 63;
  const long i = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (i >= a.N) return;
  const T pi = a.Ci[i];
  T score = T(0);
  if (pi >= a.cthr) {  // (uniform per wavefront)
    const T omp = R::add(T(1), -pi);
    for (long c0 = 0; c0 < a.Mc; c0 += 64) {
      const long c = c0 + lane;
      const long j = a.h * a.Mc + (c < a.Mc ? c : a.Mc - 1);
      const T pj = a.Cj[j];
      T term = T(0);
      if (c < a.Mc && pj >= a.cthr) {
        const T pij = a.Cij[i * a.M + j];
        T wij;
        if (a.W) {
          wij = a.W[i * a.M + j];
        } else {
          const T num = pij > a.cthr4 ? pij : a.cthr4;  // cthr^4 as well when pij is NaN
          wij = accurate_log<T>(R::div(num, R::mul(pi, pj)));
        }
        const T d = R::add(pj, -pij);
        const T yy = R::div(d, R::mul(omp, pj));
        term = R::add(R::mul(pij, wij), R::mul(d, accurate_log<T>(yy)));
      }
      // columns past the hypercolumn and columns below the threshold contribute an exact zero
#pragma unroll
      for (int k = 0; k < 64; k++) {
        T tk;
        if constexpr (sizeof(T) == 4) {
          tk = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(term), k));
        } else {
          const long long b = __double_as_longlong(term);
          const int lo = __builtin_amdgcn_readlane((int)(b & 0xffffffffLL), k);
          const int hi = __builtin_amdgcn_readlane((int)(b >> 32), k);
          tk = __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
        }
        score = R::add(score, tk);
      }
    }
  }
  int cs = 0;
  for (long g = lane; g < a.H; g += 64) cs += a.wmask[i * a.H + g];
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) cs += __shfl_xor(cs, o);
  if (lane == 0) {
    a.nom[i] = score;
    a.csum[i] = cs;
  }
}

template <typename T>
struct Cand {
  T val;
  long idx;  // -1: none
};

// a sequential ascending scan with ">=" keeps the later of two equal maxima
template <typename T>
__device__ __forceinline__ Cand<T> better_max(Cand<T> a, Cand<T> b) {
  if (a.idx < 0) return b;
  if (b.idx < 0) return a;
  if (b.val > a.val || (b.val == a.val && b.idx > a.idx)) return b;
  return a;
}
template <typename T>
__device__ __forceinline__ Cand<T> better_min(Cand<T> a, Cand<T> b) {
  if (a.idx < 0) return b;
  if (b.idx < 0) return a;
  if (b.val < a.val || (b.val == a.val && b.idx > a.idx)) return b;
  return a;
}

template <typename T>
__global__ __launch_bounds__(1024) void k_mask_swap(MaskArgs<T> a) {
  __shared__ Cand<T> smax[16], smin[16];
  __shared__ long sfirst0[16], sfirst1[16];
  __shared__ int sstop;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  for (long it = 0; it < a.iterations; it++) {
    Cand<T> cmax{T(0), -1}, cmin{T(0), -1};
    long first0 = a.N, first1 = a.N;  // first candidate rows (for the NaN rule)
    for (long i = tid; i < a.N; i += 1024) {
      const uint8_t m = a.wmask[i * a.H + a.h];
      if (m > 1) continue;
      const T s = (T)((double)a.nom[i] / (1.0 + (double)(T)a.csum[i]));
      if (m == 0) {
        first0 = i < first0 ? i : first0;
        if (s == s) cmax = better_max<T>(cmax, Cand<T>{s, i});
      } else {
        first1 = i < first1 ? i : first1;
        if (s == s) cmin = better_min<T>(cmin, Cand<T>{s, i});
      }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      Cand<T> o1{__shfl_xor(cmax.val, o), __shfl_xor(cmax.idx, o)};
      cmax = better_max<T>(cmax, o1);
      Cand<T> o2{__shfl_xor(cmin.val, o), __shfl_xor(cmin.idx, o)};
      cmin = better_min<T>(cmin, o2);
      const long f0 = __shfl_xor(first0, o), f1 = __shfl_xor(first1, o);
      first0 = f0 < first0 ? f0 : first0;
      first1 = f1 < first1 ? f1 : first1;
    }
    if (lane == 0) {
      smax[wv] = cmax;
      smin[wv] = cmin;
      sfirst0[wv] = first0;
      sfirst1[wv] = first1;
    }
    __syncthreads();
    if (tid == 0) {
      for (int k = 1; k < 16; k++) {
        cmax = better_max<T>(cmax, smax[k]);
        cmin = better_min<T>(cmin, smin[k]);
        first0 = sfirst0[k] < first0 ? sfirst0[k] : first0;
        first1 = sfirst1[k] < first1 ? sfirst1[k] : first1;
      }
      int stop = 0;
      if (first0 >= a.N || first1 >= a.N) {
        stop = 1;  // no silent or no active row
      } else {
        const T sf0 = (T)((double)a.nom[first0] / (1.0 + (double)(T)a.csum[first0]));
        const T sf1 = (T)((double)a.nom[first1] / (1.0 + (double)(T)a.csum[first1]));
        long imax0 = cmax.idx, imin1 = cmin.idx;
        T vmax0 = cmax.val, vmin1 = cmin.val;
        if (sf0 != sf0 || imax0 < 0) { imax0 = first0; vmax0 = sf0; }
        if (sf1 != sf1 || imin1 < 0) { imin1 = first1; vmin1 = sf1; }
        if (vmax0 < vmin1) {
          stop = 1;
        } else {
          a.wmask[imax0 * a.H + a.h] = 1;
          a.wmask[imin1 * a.H + a.h] = 0;
          a.csum[imax0] += 1;
          a.csum[imin1] -= 1;
        }
      }
      sstop = stop;
      __threadfence_block();
    }
    __syncthreads();
    if (sstop) break;
    __syncthreads();
  }
}

// Step 4 (mask_rows_block / k_mask_rows): the list of connected rows of a hypercolumn, which the forward
//   pass over connected rows walks:  rows[h * cap + 0 .. cnt_h) = ascending indices i with
//   wmask[i, h] != 0, the rest of the cap entries -1; row_cnt[h] = cnt_h.  One workgroup of NT threads
//   per hypercolumn; entries beyond `cap` are dropped (the host sizes cap from the column counts, so
//   none are).  Each wavefront takes a contiguous run of rows, 64 at a time: a ballot gives a row's
//   position among its 64, the wavefronts' totals meet in LDS (one barrier), and a second walk over the
//   same mask bytes writes the entries.
template <int NT = 256>
__device__ __forceinline__ void mask_rows_block(int *rows, int *row_cnt, const uint8_t *wmask, long N, long H,
                                                long cap, long h) {
  constexpr int NWV = NT / 64;
  __shared__ int wtot[NWV];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const long seg = ((N + NWV - 1) / NWV + 63) / 64 * 64;
  const long lo = wv * seg, hi = lo + seg < N ? lo + seg : N;
  int cnt = 0;
  for (long i0 = lo; i0 < hi; i0 += 64) {
    const long i = i0 + lane;
    cnt += __popcll(__ballot(i < hi && wmask[i * H + h] != 0));
  }
  if (lane == 0) wtot[wv] = cnt;
  __syncthreads();
  long pos = 0, total = 0;
#pragma unroll
  for (int u = 0; u < NWV; u++) {
    const int t = wtot[u];
    pos += u < wv ? t : 0;
    total += t;
  }
  int *list = rows + h * cap;
  for (long i0 = lo; i0 < hi; i0 += 64) {
    const long i = i0 + lane;
    const bool on = i < hi && wmask[i * H + h] != 0;
    const unsigned long long b = __ballot(on);
    const long at = pos + __popcll(b & ((1ull << lane) - 1));
    if (on && at < cap) list[at] = (int)i;
    pos += __popcll(b);
  }
  if (total > cap) total = cap;
  for (long k = total + threadIdx.x; k < cap; k += NT) list[k] = -1;
  if (threadIdx.x == 0) row_cnt[h] = (int)total;
}
// hypercolumns h0 .. h0 + gridDim.x - 1  (a template only so that the header can be included from several
// translation units)
template <int = 0>
__global__ __launch_bounds__(256) void k_mask_rows(int *rows, int *row_cnt, const uint8_t *wmask, long N,
                                                   long H, long cap, long h0) {
  mask_rows_block(rows, row_cnt, wmask, N, H, cap, h0 + blockIdx.x);
}

// Step 3; with a row list (rows != nullptr) one extra workgroup, the last, does step 4 for hypercolumn h
// in the same launch.
template <typename T>
__global__ __launch_bounds__(256) void k_mask_fix_weights(T *W, const uint8_t *wmask, const T *Ci,
                                                          const T *Cj, const T *Cij, T cthr, T cthr4,
                                                          long N, long M, long H, long Mc, long h, int *rows,
                                                          int *row_cnt, long cap) {
  if (rows != nullptr && blockIdx.x == gridDim.x - 1) {  // uniform over the workgroup
    mask_rows_block(rows, row_cnt, wmask, N, H, cap, h);
    return;
  }
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= N * Mc) return;
  const long i = e / Mc;
  const long j = h * Mc + (e - i * Mc);
  T wgt = T(0);
  if (wmask[i * H + h] != 0)
    wgt = weight_from_traces<T>(Cij[i * M + j], trace_reciprocal<T>(Ci[i], cthr),
                                trace_reciprocal<T>(Cj[j], cthr), cthr4);
  W[i * M + j] = wgt;
}

// =====================================================================================================
// Classification: first maximal index per row (np.argmax), optional comparison with one-hot labels.
// _cpu_base_backend.py:239-241.  One wavefront per row.
// =====================================================================================================
template <typename T>
__device__ __forceinline__ long wave_argmax_first(const T *row, long M, int lane) {
  T best = T(0);
  long bi = -1;
  constexpr int U = 8;  // loads in flight per lane before the (ordered) comparisons
  for (long j0 = lane; j0 < M; j0 += 64 * U) {
    T v[U];
#pragma unroll
    for (int u = 0; u < U; u++) v[u] = row[j0 + 64 * u < M ? j0 + 64 * u : M - 1];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const long j = j0 + 64 * u;
      if (j < M && (bi < 0 || v[u] > best)) {
        best = v[u];
        bi = j;
      }
    }
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    const T ov = __shfl_xor(best, o);
    const long oi = __shfl_xor(bi, o);
    if (oi >= 0 && (bi < 0 || ov > best || (ov == best && oi < bi))) {
      best = ov;
      bi = oi;
    }
  }
  return bi;
}

template <typename T>
__global__ __launch_bounds__(256) void k_argmax_rows(const T *act, const T *labels, long B, long M,
                                                     int32_t *pred, unsigned long long *correct) {
  const int lane = threadIdx.x & 63;
  const long b = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (b >= B) return;
  const long pa = wave_argmax_first<T>(act + b * M, M, lane);
  if (lane == 0 && pred) pred[b] = (int32_t)pa;
  if (labels) {
    const long pl = wave_argmax_first<T>(labels + b * M, M, lane);
    if (lane == 0 && pa == pl) atomicAdd(correct, 1ull);
  }
}

// dst[r, :] = src[idx[r], :]   (images[idx, :], _cpu_base_backend.py:258-260)
template <typename T>
__global__ __launch_bounds__(256) void k_gather_rows(T *dst, const T *src, const int64_t *idx, long rows,
                                                     long cols) {
  const long r = blockIdx.x;
  if (r >= rows) return;
  const T *s = src + idx[r] * cols;
  T *d = dst + r * cols;
  for (long c = threadIdx.x; c < cols; c += 256) d[c] = s[c];
}

// The same rows in blocks of 16, column-major inside a block:  dst[(r / 16) * cols + c][r % 16] =
// src[idx[r], c]  (idx == nullptr: src[r, c]); rows >= `rows` of the last block are written as zero.
// In this layout the 16 batch rows of a forward tile lie side by side for every input column, so a
// column picked by index costs one 64-byte access instead of 16 scattered ones.  One workgroup per block;
// a thread reads 16 elements of one column (coalesced across threads) and writes them as one run.
// plain (optional): the same rows in their plain layout, plain[r, :] = src[idx[r], :], from the same read.
template <typename T>
__global__ __launch_bounds__(256) void k_gather_rows_blocked(T *dst, T *plain, const T *src,
                                                             const int64_t *idx, long rows, long cols) {
  const long r0 = (long)blockIdx.x * 16;
  const T *s[16];
#pragma unroll
  for (int k = 0; k < 16; k++) {
    const long r = r0 + k;
    s[k] = r < rows ? src + (idx ? idx[r] : r) * cols : nullptr;
  }
  T *d = dst + (long)blockIdx.x * cols * 16;
  for (long c = threadIdx.x; c < cols; c += 256) {
    T v[16];
#pragma unroll
    for (int k = 0; k < 16; k++) v[k] = s[k] ? s[k][c] : T(0);
#pragma unroll
    for (int k = 0; k < 16; k++) d[c * 16 + k] = v[k];
    if (plain) {
#pragma unroll
      for (int k = 0; k < 16; k++)
        if (s[k]) plain[(r0 + k) * cols + c] = v[k];
    }
  }
}

// Matrix-core probe: every wavefront issues `iters` rounds of eight independent 16x16x4 MFMAs (nothing else
// in the loop), so launches / time gives the rate the matrix cores reach on this element type in practice.
template <typename T>
__global__ __launch_bounds__(256) void k_mfma_probe(T *sink, long iters) {
  using R = Real<T>;
  typename R::acc_t acc[8];
#pragma unroll
  for (int k = 0; k < 8; k++) acc[k] = typename R::acc_t{T(k), 0, 0, 0};
  const T a = T(1) + T(threadIdx.x) * T(1e-6), b = T(1) - T(threadIdx.x) * T(1e-6);
  for (long i = 0; i < iters; i++) {
#pragma unroll
    for (int k = 0; k < 8; k++) acc[k] = R::mfma(a, b, acc[k]);
  }
  T s = T(0);
#pragma unroll
  for (int k = 0; k < 8; k++) s += acc[k][0] + acc[k][1] + acc[k][2] + acc[k][3];
  if (s == T(-1)) sink[0] = s;  // never true: keeps the loop
}

// The same with the 4x4x4 form of the fp64 MFMA (four independent 4x4x4 products per instruction): sixteen
// independent accumulators, 16 * iters instructions per wavefront.  On gfx950 this form issues at the
// published fp64 matrix rate, the 16x16x4 form at two thirds of it.
template <int UNUSED = 0>
__global__ __launch_bounds__(256) void k_mfma_probe_f64_4x4x4(double *sink, long iters) {
  double acc[16];
#pragma unroll
  for (int k = 0; k < 16; k++) acc[k] = (double)k;
  const double a = 1.0 + threadIdx.x * 1e-6, b = 1.0 - threadIdx.x * 1e-6;
  for (long i = 0; i < iters; i++) {
#pragma unroll
    for (int k = 0; k < 16; k++) acc[k] = __builtin_amdgcn_mfma_f64_4x4x4f64(a, b, acc[k], 0, 0, 0);
  }
  double s = 0;
#pragma unroll
  for (int k = 0; k < 16; k++) s += acc[k];
  if (s == -1.0) sink[0] = s;  // never true: keeps the loop
}

template <int UNUSED = 0>
__global__ __launch_bounds__(256) void k_fill_bytes(uint8_t *dst, uint8_t value, size_t bytes) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < bytes; e += stride) dst[e] = value;
}

template <typename T>
__global__ __launch_bounds__(256) void k_fill(T *dst, T value, size_t n) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n; e += stride) dst[e] = value;
}

// Two short arrays copied in one launch (the new Ci and Cj of the per-function training entry points).
template <typename T>
__global__ __launch_bounds__(256) void k_copy_pair(T *dst1, const T *src1, size_t n1, T *dst2, const T *src2,
                                                   size_t n2) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n1 + n2; e += stride) {
    if (e < n1) dst1[e] = src1[e];
    else dst2[e - n1] = src2[e - n1];
  }
}

}  // namespace sb

#include "sb_k_forward.hpp"
#include "sb_k_mask_swap.hpp"
