// gfx950 kernels of the BCPNN layer step.  One wavefront = 64 lanes; lane = 16*q + p throughout.
//
// Reference semantics restated by each kernel are cited as file:line of the reference checkout
// ("omp.cc" = BCPNN/backend/_kernels/kernels_openmp_internal.cc).
#pragma once
#include "sb_common.hpp"

namespace sb {

// =====================================================================================================
// Forward: act = softmax_per_hypercolumn(x . W + bias)            omp.cc:70-87 + kernels_numpy.py:13-25
//
// A workgroup of 4 wavefronts owns 16 batch rows x one column tile (one whole hypercolumn when FUSE,
// NG*16*VW arbitrary columns otherwise).  The 4 wavefronts split the reduction dimension N in
// interleaved chunks of 4*VW; each runs 16x16x4 MFMAs with
//   A = x   : lane (p,q) loads VW consecutive k of batch row b0+p      -> VW MFMA steps
//   B = W   : lane (p,q) loads VW consecutive columns of W row k       -> VW column blocks
// so one 16-byte load of x and VW*NG 16-byte loads of W feed VW*VW*NG MFMAs.  Column block c of
// group g holds columns j0 + g*16*VW + VW*p + c (interleaved), which makes every result vector
// {c = 0..VW-1} VW consecutive columns.  Partial tiles are summed through LDS in a fixed order
// ((w0+w2)+(w1+w3)), then 16 threads per row add the bias and, when FUSE, do the softmax.
// =====================================================================================================
template <typename T>
struct ForwardArgs {
  T *act;
  const T *x;
  const T *W;
  const T *bias;
  long B, N, M, Mc;
};

template <typename T, int NG, bool FUSE, bool VEC>
__global__ __launch_bounds__(256) void k_forward(ForwardArgs<T> a) {
  constexpr int VW = Real<T>::VW;
  constexpr int GW = 16 * VW;
  constexpr int CP = NG * GW + VW;
  using acc_t = typename Real<T>::acc_t;
  using vec_t = typename Real<T>::vec_t;
  __shared__ __attribute__((aligned(16))) T red[2][16][CP];

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, p = lane & 15, q = lane >> 4;
  const long b0 = (long)blockIdx.y * 16;
  const long j0 = FUSE ? (long)blockIdx.x * a.Mc : (long)blockIdx.x * (NG * GW);
  const long jend = FUSE ? j0 + a.Mc : (j0 + NG * GW < a.M ? j0 + NG * GW : a.M);
  const long nchunks = (a.N + 4 * VW - 1) / (4 * VW);
  const bool row_ok = (b0 + p) < a.B;
  const T *xrow = a.x + (b0 + p) * a.N;

  acc_t acc[NG][VW];
#pragma unroll
  for (int g = 0; g < NG; g++)
#pragma unroll
    for (int c = 0; c < VW; c++) acc[g][c] = acc_t{0, 0, 0, 0};

  T xa[VW], xb[VW];
  T wa[VW][NG][VW], wb[VW][NG][VW];

  auto load_chunk = [&](long kc, T(&xo)[VW], T(&wo)[VW][NG][VW]) {
    const long kk = kc * (4 * VW) + VW * q;
    const bool ok = kc < nchunks;
    load_vw<T, VEC>(xo, xrow, kk, a.N, row_ok && ok);
#pragma unroll
    for (int s = 0; s < VW; s++) {
      const long krow = kk + s;
      const bool kok = ok && krow < a.N;
      const T *wrow = a.W + krow * a.M;
#pragma unroll
      for (int g = 0; g < NG; g++) load_vw<T, VEC>(wo[s][g], wrow, j0 + g * GW + VW * p, jend, kok);
    }
  };
  auto compute = [&](const T(&xi)[VW], const T(&wi)[VW][NG][VW]) {
#pragma unroll
    for (int s = 0; s < VW; s++)
#pragma unroll
      for (int g = 0; g < NG; g++)
#pragma unroll
        for (int c = 0; c < VW; c++) acc[g][c] = Real<T>::mfma(xi[s], wi[s][g][c], acc[g][c]);
  };

  load_chunk(w, xa, wa);
  for (long kc = w; kc < nchunks; kc += 8) {
    load_chunk(kc + 4, xb, wb);
    compute(xa, wa);
    load_chunk(kc + 8, xa, wa);
    compute(xb, wb);
  }

  // ---- cross-wavefront sum through LDS: slots 0/1 end up holding (w0+w2) and (w1+w3)
  if (w >= 2) {
#pragma unroll
    for (int g = 0; g < NG; g++)
#pragma unroll
      for (int v = 0; v < 4; v++) {
        vec_t t;
#pragma unroll
        for (int c = 0; c < VW; c++) t[c] = acc[g][c][v];
        *reinterpret_cast<vec_t *>(&red[w - 2][Real<T>::acc_row(q, v)][g * GW + VW * p]) = t;
      }
  }
  __syncthreads();
  if (w < 2) {
#pragma unroll
    for (int g = 0; g < NG; g++)
#pragma unroll
      for (int v = 0; v < 4; v++) {
        vec_t *slot = reinterpret_cast<vec_t *>(&red[w][Real<T>::acc_row(q, v)][g * GW + VW * p]);
        vec_t t = *slot;
#pragma unroll
        for (int c = 0; c < VW; c++) t[c] = acc[g][c][v] + t[c];
        *slot = t;
      }
  }
  __syncthreads();

  // ---- bias (+ softmax): 16 threads per batch row, thread handles columns l16, l16+16, ...
  const int row = tid >> 4, l16 = tid & 15;
  const long ncol = jend - j0;
  constexpr int PER = NG * VW;
  T vals[PER];
  T mx = -INFINITY;
#pragma unroll
  for (int t = 0; t < PER; t++) {
    const long col = l16 + 16 * t;
    vals[t] = T(0);
    if (col < ncol) {
      vals[t] = (red[0][row][col] + red[1][row][col]) + a.bias[j0 + col];
      mx = vals[t] > mx ? vals[t] : mx;
    }
  }
  if (FUSE) {
#pragma unroll
    for (int o = 8; o >= 1; o >>= 1) {
      const T other = __shfl_xor(mx, o);
      mx = other > mx ? other : mx;
    }
    T sum = T(0);
#pragma unroll
    for (int t = 0; t < PER; t++) {
      const long col = l16 + 16 * t;
      if (col < ncol) {
        vals[t] = Real<T>::exp_(vals[t] - mx);
        sum += vals[t];
      }
    }
#pragma unroll
    for (int o = 8; o >= 1; o >>= 1) sum += __shfl_xor(sum, o);
#pragma unroll
    for (int t = 0; t < PER; t++) vals[t] = vals[t] / sum;
  }
  if (b0 + row < a.B) {
    T *out = a.act + (b0 + row) * a.M + j0;
#pragma unroll
    for (int t = 0; t < PER; t++) {
      const long col = l16 + 16 * t;
      if (col < ncol) out[col] = vals[t];
    }
  }
}

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

// =====================================================================================================
// Ci / Cj moving averages (+ bias of a plastic layer)                   omp.cc:106-156, 222-246
// One thread per trace element; the batch sum runs b = 0..B-1 in REAL without FMA contraction, then
// /B, *taupdt, C*(1-taupdt) + tmp, max(0, .) -- the reference's order, so Ci and Cj are bit-exact
// against a strict-IEEE build of it.
// =====================================================================================================
template <typename T>
struct CountersArgs {
  const T *x;  // [B,N]
  const T *y;  // [B,M]
  T *Ci, *Cj;
  long B, N, M;
  T tau, omt, fB;
  int bias_mode;  // 0: leave bias alone; 1: update_bias_regularized on the fresh Cj
  T *bias, *kbi;
  T cthr, khalf, pmin, taubdt;
};

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

template <typename T>
__global__ __launch_bounds__(256) void k_counters(CountersArgs<T> a) {
  using R = Real<T>;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const bool is_i = idx < a.N;
  const long col = is_i ? idx : idx - a.N;
  const long ld = is_i ? a.N : a.M;
  if (!is_i && col >= a.M) return;
  const T *src = (is_i ? a.x : a.y) + col;
  T s = T(0);
  for (long b = 0; b < a.B; b++) s = R::add(s, src[b * ld]);
  s = R::div(s, a.fB);
  s = R::mul(s, a.tau);
  T *C = is_i ? a.Ci : a.Cj;
  T c = R::add(R::mul(C[col], a.omt), s);
  c = c > T(0) ? c : T(0);
  C[col] = c;
  if (!is_i && a.bias_mode == 1) {
    T kb = a.kbi[col];
    a.bias[col] = bias_regularized<T>(c, kb, a.cthr, a.khalf, a.pmin, a.taubdt);
    a.kbi[col] = kb;
  }
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

// =====================================================================================================
// Cij moving average as a rank-B MFMA update with the decay, clamp, weight recompute and mask apply in
// the epilogue:                                                          omp.cc:158-201, 322-335
//   Cij <- max(0, Cij*(1-taupdt) + (x^T y / B) * taupdt)
//   W   <- wmask ? log(max(Cij, cthr^4) / (Ci*Cj)) : 0     (0 as well where Ci < cthr or Cj < cthr)
// Ci and Cj are this step's already-updated traces.
//
// A wavefront owns a (RX*16*VW) x (RY*16*VW) tile of Cij for the whole batch (K = B).  Both operands
// are "k-major" in memory (x[b][i], y[b][j]), exactly the MFMA operand layout, so they are loaded
// straight from L2 into registers: lane (p,q) loads VW consecutive i (resp. j) of batch row 4s+q.
// Block (r,c) of the tile then holds rows i0 + VW*p16 + r and columns j0 + VW*p + c, which turns every
// Cij / W access of the epilogue into one 16-byte vector per lane (256 contiguous bytes per 16 lanes).
// With PRE the Cij tile is requested before the K loop so HBM latency hides behind the MFMAs.
// =====================================================================================================
template <typename T>
struct TraceArgs {
  const T *x;  // [B,N]
  const T *y;  // [B,M]
  T *Cij;
  T *W;
  const T *Ci;
  const T *Cj;
  const uint8_t *wmask;  // [N,H] or nullptr (no mask: every synapse active)
  long B, N, M, H, Mc;
  T tau, omt, invB, cthr, cthr4;
};

template <typename T, int RX, int RY, bool VEC, bool PRE>
__global__ __launch_bounds__(256) void k_trace_weights(TraceArgs<T> a) {
  constexpr int VW = Real<T>::VW;
  constexpr int GW = 16 * VW;
  constexpr int TI = RX * GW, TJ = RY * GW;
  using acc_t = typename Real<T>::acc_t;

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, p = lane & 15, q = lane >> 4;
  const long i0 = ((long)blockIdx.y * 2 + (w >> 1)) * TI;
  const long j0 = ((long)blockIdx.x * 2 + (w & 1)) * TJ;
  if (i0 >= a.N || j0 >= a.M) return;  // wavefront-uniform; the kernel has no barriers

  T cpre[PRE ? RX : 1][VW][4][PRE ? RY : 1][VW];
  if (PRE) {
#pragma unroll
    for (int rx = 0; rx < RX; rx++)
#pragma unroll
      for (int r = 0; r < VW; r++)
#pragma unroll
        for (int v = 0; v < 4; v++) {
          const long row = i0 + rx * GW + VW * Real<T>::acc_row(q, v) + r;
#pragma unroll
          for (int ry = 0; ry < RY; ry++)
            load_vw<T, VEC>(cpre[rx][r][v][ry], a.Cij + row * a.M, j0 + ry * GW + VW * p, a.M,
                            row < a.N);
        }
  }

  acc_t acc[RX * VW][RY * VW];
#pragma unroll
  for (int i = 0; i < RX * VW; i++)
#pragma unroll
    for (int j = 0; j < RY * VW; j++) acc[i][j] = acc_t{0, 0, 0, 0};

  constexpr int PF = 4;
  T xr[PF][RX][VW], yr[PF][RY][VW];
  auto load_step = [&](long s, T(&xo)[RX][VW], T(&yo)[RY][VW]) {
    const long b = 4 * s + q;
    const bool ok = b < a.B;
    const T *xrow = a.x + b * a.N;
    const T *yrow = a.y + b * a.M;
#pragma unroll
    for (int rx = 0; rx < RX; rx++) load_vw<T, VEC>(xo[rx], xrow, i0 + rx * GW + VW * p, a.N, ok);
#pragma unroll
    for (int ry = 0; ry < RY; ry++) load_vw<T, VEC>(yo[ry], yrow, j0 + ry * GW + VW * p, a.M, ok);
  };
#pragma unroll
  for (int u = 0; u < PF; u++) load_step(u, xr[u], yr[u]);
  const long nsteps = (a.B + 3) / 4;
  for (long s0 = 0; s0 < nsteps; s0 += PF) {
#pragma unroll
    for (int u = 0; u < PF; u++) {
      T xa[RX][VW], ya[RY][VW];
#pragma unroll
      for (int rx = 0; rx < RX; rx++)
#pragma unroll
        for (int e = 0; e < VW; e++) xa[rx][e] = xr[u][rx][e];
#pragma unroll
      for (int ry = 0; ry < RY; ry++)
#pragma unroll
        for (int e = 0; e < VW; e++) ya[ry][e] = yr[u][ry][e];
      load_step(s0 + u + PF, xr[u], yr[u]);
#pragma unroll
      for (int rx = 0; rx < RX; rx++)
#pragma unroll
        for (int r = 0; r < VW; r++)
#pragma unroll
          for (int ry = 0; ry < RY; ry++)
#pragma unroll
            for (int c = 0; c < VW; c++)
              acc[rx * VW + r][ry * VW + c] =
                  Real<T>::mfma(xa[rx][r], ya[ry][c], acc[rx * VW + r][ry * VW + c]);
    }
  }

  // ---- epilogue
  T rci_l[RX][VW], rcj_l[RY][VW];
  uint32_t hc_l[RY][VW];
#pragma unroll
  for (int rx = 0; rx < RX; rx++)
#pragma unroll
    for (int r = 0; r < VW; r++) {
      const long row = i0 + rx * GW + VW * p + r;
      rci_l[rx][r] = trace_reciprocal<T>(row < a.N ? a.Ci[row] : T(1), a.cthr);
    }
#pragma unroll
  for (int ry = 0; ry < RY; ry++)
#pragma unroll
    for (int c = 0; c < VW; c++) {
      const long col = j0 + ry * GW + VW * p + c;
      rcj_l[ry][c] = trace_reciprocal<T>(col < a.M ? a.Cj[col] : T(1), a.cthr);
      hc_l[ry][c] = col < a.M ? (uint32_t)col / (uint32_t)a.Mc : 0u;
    }

#pragma unroll
  for (int rx = 0; rx < RX; rx++)
#pragma unroll
    for (int r = 0; r < VW; r++)
#pragma unroll
      for (int v = 0; v < 4; v++) {
        const int p16 = Real<T>::acc_row(q, v);
        const long row = i0 + rx * GW + VW * p16 + r;
        const T rci = __shfl(rci_l[rx][r], p16);
        if (row < a.N) {
          T *crow = a.Cij + row * a.M;
          T *wrow = a.W + row * a.M;
          const uint8_t *mrow = a.wmask ? a.wmask + row * a.H : nullptr;
#pragma unroll
          for (int ry = 0; ry < RY; ry++) {
            const long col = j0 + ry * GW + VW * p;
            T cv[VW], wv[VW];
            if (PRE) {
#pragma unroll
              for (int c = 0; c < VW; c++) cv[c] = cpre[rx][r][v][ry][c];
            } else {
              load_vw<T, VEC>(cv, crow, col, a.M, true);
            }
#pragma unroll
            for (int c = 0; c < VW; c++) {
              T t = acc[rx * VW + r][ry * VW + c][v] * a.invB;
              t = t * a.tau;
              T cn = cv[c] * a.omt + t;
              cn = cn > T(0) ? cn : T(0);
              cv[c] = cn;
              T wgt = weight_from_traces<T>(cn, rci, rcj_l[ry][c], a.cthr4);
              if (mrow && col + c < a.M && mrow[hc_l[ry][c]] == 0) wgt = T(0);
              wv[c] = wgt;
            }
            store_vw<T, VEC>(cv, crow, col, a.M);
            store_vw<T, VEC>(wv, wrow, col, a.M);
          }
        }
      }
}

// omp.cc:322-335
template <typename T>
__global__ __launch_bounds__(256) void k_apply_mask(T *W, const uint8_t *wmask, long N, long M, long H,
                                                    long Mc) {
  const long total = N * M;
  const long stride = (long)gridDim.x * 256;
  for (long e = (long)blockIdx.x * 256 + threadIdx.x; e < total; e += stride) {
    const long i = e / M;
    const long j = e - i * M;
    if (wmask[i * H + j / Mc] == 0) W[e] = T(0);
  }
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
};

template <typename T>
__global__ __launch_bounds__(256) void k_mask_scores(MaskArgs<T> a) {
  const int lane = threadIdx.x & 63;
  const long i = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (i >= a.N) return;
  const T pi = a.Ci[i];
  const T rci = trace_reciprocal<T>(pi, a.cthr);
  T score = T(0);
  if (pi >= a.cthr) {
    for (long c = lane; c < a.Mc; c += 64) {
      const long j = a.h * a.Mc + c;
      const T pj = a.Cj[j];
      if (pj >= a.cthr) {
        const T pij = a.Cij[i * a.M + j];
        const T wij = a.W ? a.W[i * a.M + j]
                          : weight_from_traces<T>(pij, rci, trace_reciprocal<T>(pj, a.cthr), a.cthr4);
        const T xx = (T(1) - pi) * pj;
        const T yy = (pj - pij) / xx;
        score += pij * wij + (pj - pij) * Real<T>::log_(yy);
      }
    }
  }
  int cs = 0;
  for (long g = lane; g < a.H; g += 64) cs += a.wmask[i * a.H + g];
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    score += __shfl_xor(score, o);
    cs += __shfl_xor(cs, o);
  }
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

template <typename T>
__global__ __launch_bounds__(256) void k_mask_fix_weights(T *W, const uint8_t *wmask, const T *Ci,
                                                          const T *Cj, const T *Cij, T cthr, T cthr4,
                                                          long N, long M, long H, long Mc, long h) {
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
  for (long j = lane; j < M; j += 64) {
    const T v = row[j];
    if (bi < 0 || v > best) {
      best = v;
      bi = j;
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

}  // namespace sb
