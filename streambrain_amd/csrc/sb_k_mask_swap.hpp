// Register-resident variant of the greedy swap loop of the mask rewiring (omp.cc:289-315, where
// "omp.cc" = BCPNN/backend/_kernels/kernels_openmp_internal.cc of the reference) for layers with at
// most NT*R input rows: one small workgroup of NT threads, thread t owns rows t, t+NT, ...; score
// nominators, connection counts, mask bits and scores stay in registers over all iterations.  Per
// iteration: a DPP / shuffle reduction inside each wavefront, one partial result per wavefront through
// LDS, a second reduction that leaves the decision in every lane -- one barrier.  Same decisions as
// k_mask_swap (which keeps its state in global memory and serves larger layers).
#pragma once
#include "sb_kernels.hpp"

namespace sb {

template <typename T>
__device__ __forceinline__ T mask_score(T nom, int csum) {
  // nominator / (1.0 + (REAL)csum): formed in double and narrowed, as the reference's expression
  return (T)((double)nom / (1.0 + (double)(T)csum));
}

// candidate row: score and row index (-1: none)
template <typename T>
struct RowCand {
  T val;
  int idx;
};
template <typename T>
__device__ __forceinline__ RowCand<T> shfl_xor_cand(RowCand<T> c, int o) {
  return RowCand<T>{__shfl_xor(c.val, o), __shfl_xor(c.idx, o)};
}
// Exchange inside a row of 16 lanes with data-parallel-primitive moves (no LDS round trip).  The four
// controls below -- swap neighbours, swap pairs, mirror each half row, mirror the row -- applied in
// turn with a commutative pick leave the row-wide result in every one of the 16 lanes.
constexpr int kDppSwap1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppSwap2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // row_half_mirror
constexpr int kDppMirror = 0x140;      // row_mirror
template <int CTRL>
__device__ __forceinline__ int dpp_move(int v) {
  return __builtin_amdgcn_update_dpp(v, v, CTRL, 0xF, 0xF, false);
}
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(dpp_move<CTRL>(__float_as_int(v)));
}
template <int CTRL>
__device__ __forceinline__ double dpp_move(double v) {
  const long long b = __double_as_longlong(v);
  const int lo = dpp_move<CTRL>((int)(b & 0xffffffffLL)), hi = dpp_move<CTRL>((int)(b >> 32));
  return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}
template <int CTRL, typename T>
__device__ __forceinline__ RowCand<T> dpp_cand(RowCand<T> c) {
  return RowCand<T>{dpp_move<CTRL>(c.val), dpp_move<CTRL>(c.idx)};
}
// reduce over the 16 lanes of each row with `pick`; every lane of the row ends with the result
#define SB_ROW_REDUCE(pick, c)                        \
  do {                                                \
    c = pick(c, dpp_cand<kDppSwap1, T>(c));           \
    c = pick(c, dpp_cand<kDppSwap2, T>(c));           \
    c = pick(c, dpp_cand<kDppHalfMirror, T>(c));      \
    c = pick(c, dpp_cand<kDppMirror, T>(c));          \
  } while (0)
// ascending scan with ">=" keeps the later of two equal maxima; with "<=" the later of two equal minima
template <typename T>
__device__ __forceinline__ RowCand<T> pick_max(RowCand<T> a, RowCand<T> b) {
  const bool take = b.idx >= 0 && (a.idx < 0 || b.val > a.val || (b.val == a.val && b.idx > a.idx));
  return take ? b : a;
}
template <typename T>
__device__ __forceinline__ RowCand<T> pick_min(RowCand<T> a, RowCand<T> b) {
  const bool take = b.idx >= 0 && (a.idx < 0 || b.val < a.val || (b.val == a.val && b.idx > a.idx));
  return take ? b : a;
}
template <typename T>
__device__ __forceinline__ RowCand<T> pick_first(RowCand<T> a, RowCand<T> b) {
  const bool take = b.idx >= 0 && (a.idx < 0 || b.idx < a.idx);
  return take ? b : a;
}

// NT threads (a multiple of 64, at most 256: one wavefront per SIMD, so the replicated reduction code
// is not time-shared), thread t owns rows t, t+NT, ..., t+(R-1)*NT.
template <typename T, int NT, int R>
__global__ __launch_bounds__(NT) void k_mask_swap_reg(MaskArgs<T> a) {
  constexpr int NWV = NT / 64;
  static_assert(NWV == 1 || NWV == 2 || NWV == 4, "1, 2 or 4 wavefronts");
  __shared__ RowCand<T> part[2][4][NWV];  // [buffer][max0, min1, first0, first1][wavefront]
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;

  T nom[R], score[R];
  int cs[R], m[R];  // m: 0 silent, 1 active, 2 not a candidate (row out of range or odd mask value)
  bool dirty[R];
  int has_nan = 0;
#pragma unroll
  for (int k = 0; k < R; k++) {
    const long i = tid + (long)NT * k;
    dirty[k] = false;
    m[k] = 2;
    nom[k] = T(0);
    cs[k] = 0;
    if (i < a.N) {
      const uint8_t b = a.wmask[i * a.H + a.h];
      m[k] = b > 1 ? 2 : b;
      nom[k] = a.nom[i];
      cs[k] = a.csum[i];
    }
    score[k] = mask_score<T>(nom[k], cs[k]);
    has_nan |= (score[k] != score[k]) ? 1 : 0;
  }
  // NaN scores need the "first candidate" bookkeeping of the sequential scan; without any NaN (the
  // normal case; a score is NaN iff its nominator is) that half of the reduction is skipped
  const bool track_first = __syncthreads_or(has_nan) != 0;

  for (long it = 0; it < a.iterations; it++) {
    const int buf = (int)(it & 1);
    RowCand<T> cmax{T(0), -1}, cmin{T(0), -1}, f0{T(0), -1}, f1{T(0), -1};
#pragma unroll
    for (int k = 0; k < R; k++) {  // ascending row order within the thread
      const int i = tid + NT * k;
      const RowCand<T> me{score[k], i};
      const bool num = score[k] == score[k];  // a NaN never wins a comparison
      if (m[k] == 0) {
        if (track_first) f0 = pick_first<T>(f0, me);
        if (num) cmax = pick_max<T>(cmax, me);
      } else if (m[k] == 1) {
        if (track_first) f1 = pick_first<T>(f1, me);
        if (num) cmin = pick_min<T>(cmin, me);
      }
    }
    SB_ROW_REDUCE(pick_max<T>, cmax);
    SB_ROW_REDUCE(pick_min<T>, cmin);
    if (track_first) {
      SB_ROW_REDUCE(pick_first<T>, f0);
      SB_ROW_REDUCE(pick_first<T>, f1);
    }
#pragma unroll
    for (int o = 16; o <= 32; o <<= 1) {  // across the four rows of the wavefront
      cmax = pick_max<T>(cmax, shfl_xor_cand<T>(cmax, o));
      cmin = pick_min<T>(cmin, shfl_xor_cand<T>(cmin, o));
      if (track_first) {
        f0 = pick_first<T>(f0, shfl_xor_cand<T>(f0, o));
        f1 = pick_first<T>(f1, shfl_xor_cand<T>(f1, o));
      }
    }
    if (NWV > 1) {
      if (lane == 0) {
        part[buf][0][wv] = cmax;
        part[buf][1][wv] = cmin;
        part[buf][2][wv] = f0;
        part[buf][3][wv] = f1;
      }
      __syncthreads();
      // every group of NWV lanes reads the NWV partials and reduces them: all lanes get the result
      cmax = part[buf][0][lane % NWV];
      cmin = part[buf][1][lane % NWV];
      f0 = part[buf][2][lane % NWV];
      f1 = part[buf][3][lane % NWV];
      cmax = pick_max<T>(cmax, dpp_cand<kDppSwap1, T>(cmax));
      cmin = pick_min<T>(cmin, dpp_cand<kDppSwap1, T>(cmin));
      f0 = pick_first<T>(f0, dpp_cand<kDppSwap1, T>(f0));
      f1 = pick_first<T>(f1, dpp_cand<kDppSwap1, T>(f1));
      if (NWV > 2) {
        cmax = pick_max<T>(cmax, dpp_cand<kDppSwap2, T>(cmax));
        cmin = pick_min<T>(cmin, dpp_cand<kDppSwap2, T>(cmin));
        f0 = pick_first<T>(f0, dpp_cand<kDppSwap2, T>(f0));
        f1 = pick_first<T>(f1, dpp_cand<kDppSwap2, T>(f1));
      }
    }
    if (cmax.idx < 0 && f0.idx < 0) break;  // no silent row (uniform over the workgroup)
    if (cmin.idx < 0 && f1.idx < 0) break;  // no active row
    int imax0 = cmax.idx, imin1 = cmin.idx;
    T vmax0 = cmax.val, vmin1 = cmin.val;
    // a NaN score wins only when it belongs to the first candidate row (sequential >= / <= scan)
    if (track_first) {
      if (f0.val != f0.val || imax0 < 0) { imax0 = f0.idx; vmax0 = f0.val; }
      if (f1.val != f1.val || imin1 < 0) { imin1 = f1.idx; vmin1 = f1.val; }
    }
    if (vmax0 < vmin1) break;
#pragma unroll
    for (int k = 0; k < R; k++) {
      const int i = tid + NT * k;
      if (i == imax0) { m[k] = 1; cs[k] += 1; dirty[k] = true; score[k] = mask_score<T>(nom[k], cs[k]); }
      if (i == imin1) { m[k] = 0; cs[k] -= 1; dirty[k] = true; score[k] = mask_score<T>(nom[k], cs[k]); }
    }
  }
#pragma unroll
  for (int k = 0; k < R; k++) {
    const long i = tid + (long)NT * k;
    if (dirty[k]) {
      a.wmask[i * a.H + a.h] = (uint8_t)m[k];
      a.csum[i] = cs[k];
    }
  }
}

}  // namespace sb
