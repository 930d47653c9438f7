// Probability-trace kernels: Ci / Cj moving averages and the fused Cij + weight pass.
// ("omp.cc" = BCPNN/backend/_kernels/kernels_openmp_internal.cc of the reference)
#pragma once
#include "sb_common.hpp"

namespace sb {

// =====================================================================================================
// Ci / Cj moving averages (+ regularised bias of a plastic layer)          omp.cc:106-156, 222-246
//
// The batch sum of every column runs b = 0..B-1 in REAL without FMA contraction, then /B, *taupdt,
// C*(1-taupdt) + tmp, max(0, .) -- the reference's order, so Ci, Cj (and kbi) are bit-exact against a
// strict-IEEE build of it.  To keep that order and still have every load in flight at once, a
// workgroup stages a [CH rows x 64 columns] slab of the activity matrix in LDS with all 256 threads
// (coalesced 64-column rows), then 64 threads add their column top to bottom.
// =====================================================================================================
template <typename T>
__global__ __launch_bounds__(256) void k_counters(CountersArgs<T> a) {
  using R = Real<T>;
  constexpr int CH = sizeof(T) == 4 ? 128 : 64;
  __shared__ T slab[CH][64];
  const int tid = threadIdx.x, c = tid & 63, r0 = tid >> 6;
  const long nbi = (a.N + 63) / 64;
  const bool is_i = (long)blockIdx.x < nbi;
  const long col = (is_i ? (long)blockIdx.x : (long)blockIdx.x - nbi) * 64 + c;
  const long ld = is_i ? a.N : a.M;
  const T *src = is_i ? a.x : a.y;
  const bool col_ok = col < ld;
  T s = T(0);
  for (long b0 = 0; b0 < a.B; b0 += CH) {
    const long rows = a.B - b0 < CH ? a.B - b0 : CH;
#pragma unroll
    for (int r = r0; r < CH; r += 4) slab[r][c] = (r < rows && col_ok) ? src[(b0 + r) * ld + col] : T(0);
    __syncthreads();
    if (tid < 64)
      for (int r = 0; r < rows; r++) s = R::add(s, slab[r][c]);
    __syncthreads();
  }
  if (tid >= 64 || !col_ok) return;
  s = R::div(s, a.fB);
  s = R::mul(s, a.tau);
  T *C = is_i ? a.Ci : a.Cj;
  T cnew = R::add(R::mul(C[col], a.omt), s);
  cnew = cnew > T(0) ? cnew : T(0);
  C[col] = cnew;
  if (!is_i && a.bias_mode == 1) {
    T kb = a.kbi[col];
    a.bias[col] = bias_regularized<T>(cnew, kb, a.cthr, a.khalf, a.pmin, a.taubdt);
    a.kbi[col] = kb;
  }
}

// =====================================================================================================
// Cij moving average as a rank-B MFMA update with the decay, clamp, weight recompute and mask apply in
// the epilogue:                                                          omp.cc:158-201, 322-335
//   Cij <- max(0, Cij*(1-taupdt) + (x^T y / B) * taupdt)
//   W   <- wmask ? log(max(Cij, cthr^4) / (Ci*Cj)) : 0     (0 as well where Ci < cthr or Cj < cthr)
// Ci and Cj are this step's already-updated traces.
//
// A wavefront owns a (RX*16*XW) x (RY*16*YW) tile of Cij for the whole batch (K = B).  Both operands
// are "k-major" in memory (x[b][i], y[b][j]), exactly the 16x16x4 MFMA operand layout, so they go
// straight from L2 into registers: lane (p,q) loads XW consecutive i (resp. YW consecutive j) of batch
// row 4s+q.  Block (r,c) of the tile then holds rows i0 + XW*p16 + r and columns j0 + YW*p + c, which
// turns every Cij / W access of the epilogue into one YW-element vector per lane (16 lanes cover
// 16*YW contiguous elements of a row).  With PRE the Cij tile is requested before the K loop so its
// HBM latency hides behind the MFMAs.  A workgroup is 4 wavefronts in a 2 x 2 arrangement of tiles.
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
  int dbg;  // profiling experiments: bit0 skip the K loop, bit1 leave before the epilogue
};

template <typename T, int XW, int YW, int RX, int RY, bool VEC, bool PRE>
__global__ __launch_bounds__(256) void k_trace_weights(TraceArgs<T> a) {
  constexpr int GX = 16 * XW, GY = 16 * YW;
  constexpr int TI = RX * GX, TJ = RY * GY;
  constexpr int BR = RX * XW, BC = RY * YW;  // MFMA blocks per tile: BR x BC
  using acc_t = typename Real<T>::acc_t;

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, p = lane & 15, q = lane >> 4;
  const long i0 = ((long)blockIdx.y * 2 + (w >> 1)) * TI;
  const long j0 = ((long)blockIdx.x * 2 + (w & 1)) * TJ;
  if (i0 >= a.N || j0 >= a.M) return;  // wavefront-uniform; the kernel has no barriers

  T cpre[PRE ? RX : 1][XW][4][PRE ? RY : 1][YW];
  if (PRE) {
#pragma unroll
    for (int rx = 0; rx < RX; rx++)
#pragma unroll
      for (int r = 0; r < XW; r++)
#pragma unroll
        for (int v = 0; v < 4; v++) {
          const long row = i0 + rx * GX + XW * Real<T>::acc_row(q, v) + r;
#pragma unroll
          for (int ry = 0; ry < RY; ry++)
            load_w<T, YW, VEC>(cpre[rx][r][v][ry], a.Cij + row * a.M, j0 + ry * GY + YW * p, a.M,
                               row < a.N);
        }
  }

  acc_t acc[BR][BC];
#pragma unroll
  for (int i = 0; i < BR; i++)
#pragma unroll
    for (int j = 0; j < BC; j++) acc[i][j] = acc_t{0, 0, 0, 0};

  constexpr int PF = 4;  // K steps in flight
  T xr[PF][RX][XW], yr[PF][RY][YW];
  auto load_step = [&](long s, T(&xo)[RX][XW], T(&yo)[RY][YW]) {
    const long b = 4 * s + q;
    const bool ok = b < a.B;
    const T *xrow = a.x + b * a.N;
    const T *yrow = a.y + b * a.M;
#pragma unroll
    for (int rx = 0; rx < RX; rx++) load_w<T, XW, VEC>(xo[rx], xrow, i0 + rx * GX + XW * p, a.N, ok);
#pragma unroll
    for (int ry = 0; ry < RY; ry++) load_w<T, YW, VEC>(yo[ry], yrow, j0 + ry * GY + YW * p, a.M, ok);
  };
  auto mfma_step = [&](const T(&xa)[RX][XW], const T(&ya)[RY][YW]) {
#pragma unroll
    for (int rx = 0; rx < RX; rx++)
#pragma unroll
      for (int r = 0; r < XW; r++)
#pragma unroll
        for (int ry = 0; ry < RY; ry++)
#pragma unroll
          for (int c = 0; c < YW; c++)
            acc[rx * XW + r][ry * YW + c] =
                Real<T>::mfma(xa[rx][r], ya[ry][c], acc[rx * XW + r][ry * YW + c]);
  };
  const long nsteps = (a.B + 3) / 4;
  if (a.dbg & 1) {
  } else if (VEC && a.B >= 4 * PF) {
    // Lean main loop: unguarded vector loads through per-lane pointers that advance 4 batch rows per
    // step.  Rows / columns outside the matrix are redirected to a valid address; what they feed ends
    // in accumulator rows / columns that are never stored.  Steps whose 4 batch rows are not all
    // inside the batch (at most the last one) go through the guarded loader.
    const T *xp[RX], *yp[RY];
#pragma unroll
    for (int rx = 0; rx < RX; rx++) {
      long col = i0 + rx * GX + XW * p;
      if (col >= a.N) col = 0;
      xp[rx] = a.x + (long)q * a.N + col;
    }
#pragma unroll
    for (int ry = 0; ry < RY; ry++) {
      long col = j0 + ry * GY + YW * p;
      if (col >= a.M) col = 0;
      yp[ry] = a.y + (long)q * a.M + col;
    }
    const long xstep = 4 * a.N, ystep = 4 * a.M;
    auto load_fast = [&](T(&xo)[RX][XW], T(&yo)[RY][YW]) {
#pragma unroll
      for (int rx = 0; rx < RX; rx++) {
        load_w<T, XW, true>(xo[rx], xp[rx], 0, 1, true);
        xp[rx] += xstep;
      }
#pragma unroll
      for (int ry = 0; ry < RY; ry++) {
        load_w<T, YW, true>(yo[ry], yp[ry], 0, 1, true);
        yp[ry] += ystep;
      }
    };
    const long nfast = a.B / 4;  // steps with all 4 batch rows valid; nfast >= PF here
#pragma unroll
    for (int u = 0; u < PF; u++) load_fast(xr[u], yr[u]);
    long s0 = 0;
    for (; s0 + 2 * PF <= nfast; s0 += PF) {  // steady state: every refill is a fast step
#pragma unroll
      for (int u = 0; u < PF; u++) {
        T xa[RX][XW], ya[RY][YW];
#pragma unroll
        for (int rx = 0; rx < RX; rx++)
#pragma unroll
          for (int e = 0; e < XW; e++) xa[rx][e] = xr[u][rx][e];
#pragma unroll
        for (int ry = 0; ry < RY; ry++)
#pragma unroll
          for (int e = 0; e < YW; e++) ya[ry][e] = yr[u][ry][e];
        load_fast(xr[u], yr[u]);
        mfma_step(xa, ya);
      }
    }
    for (; s0 < nsteps; s0 += PF) {  // drain: refills past the fast range use the guarded loader
#pragma unroll
      for (int u = 0; u < PF; u++) {
        T xa[RX][XW], ya[RY][YW];
#pragma unroll
        for (int rx = 0; rx < RX; rx++)
#pragma unroll
          for (int e = 0; e < XW; e++) xa[rx][e] = xr[u][rx][e];
#pragma unroll
        for (int ry = 0; ry < RY; ry++)
#pragma unroll
          for (int e = 0; e < YW; e++) ya[ry][e] = yr[u][ry][e];
        const long nxt = s0 + u + PF;
        if (nxt < nfast)
          load_fast(xr[u], yr[u]);
        else
          load_step(nxt, xr[u], yr[u]);
        mfma_step(xa, ya);
      }
    }
  } else {
#pragma unroll
    for (int u = 0; u < PF; u++) load_step(u, xr[u], yr[u]);
    for (long s0 = 0; s0 < nsteps; s0 += PF) {
#pragma unroll
      for (int u = 0; u < PF; u++) {
        T xa[RX][XW], ya[RY][YW];
#pragma unroll
        for (int rx = 0; rx < RX; rx++)
#pragma unroll
          for (int e = 0; e < XW; e++) xa[rx][e] = xr[u][rx][e];
#pragma unroll
        for (int ry = 0; ry < RY; ry++)
#pragma unroll
          for (int e = 0; e < YW; e++) ya[ry][e] = yr[u][ry][e];
        load_step(s0 + u + PF, xr[u], yr[u]);
        mfma_step(xa, ya);
      }
    }
  }

  if (a.dbg & 2) {
    if (acc[0][0][0] == T(12345.678)) a.W[0] = acc[0][0][0] + cpre[0][0][0][0][0];
    return;
  }
  // ---- epilogue
  T rci_l[RX][XW], rcj_l[RY][YW];
  uint32_t hc_l[RY][YW];
  bool one_hc[RY];
#pragma unroll
  for (int rx = 0; rx < RX; rx++)
#pragma unroll
    for (int r = 0; r < XW; r++) {
      const long row = i0 + rx * GX + XW * p + r;
      rci_l[rx][r] = trace_reciprocal<T>(row < a.N ? a.Ci[row] : T(1), a.cthr);
    }
#pragma unroll
  for (int ry = 0; ry < RY; ry++) {
#pragma unroll
    for (int c = 0; c < YW; c++) {
      const long col = j0 + ry * GY + YW * p + c;
      rcj_l[ry][c] = trace_reciprocal<T>(col < a.M ? a.Cj[col] : T(1), a.cthr);
      hc_l[ry][c] = col < a.M ? (uint32_t)col / (uint32_t)a.Mc : 0u;
    }
    // the lane's YW columns usually sit in one hypercolumn: then one mask byte serves the vector
    one_hc[ry] = (j0 + ry * GY + YW * p + YW - 1 < a.M) && hc_l[ry][0] == hc_l[ry][YW - 1];
  }

#pragma unroll
  for (int rx = 0; rx < RX; rx++)
#pragma unroll
    for (int r = 0; r < XW; r++)
#pragma unroll
      for (int v = 0; v < 4; v++) {
        const int p16 = Real<T>::acc_row(q, v);
        const long row = i0 + rx * GX + XW * p16 + r;
        const T rci = __shfl(rci_l[rx][r], p16);
        if (row < a.N) {
          T *crow = a.Cij + row * a.M;
          T *wrow = a.W + row * a.M;
          const uint8_t *mrow = a.wmask ? a.wmask + row * a.H : nullptr;
#pragma unroll
          for (int ry = 0; ry < RY; ry++) {
            const long col = j0 + ry * GY + YW * p;
            T cv[YW], wv[YW];
            if (PRE) {
#pragma unroll
              for (int c = 0; c < YW; c++) cv[c] = cpre[rx][r][v][ry][c];
            } else {
              load_w<T, YW, VEC>(cv, crow, col, a.M, true);
            }
            bool on[YW];
            if (!mrow) {
#pragma unroll
              for (int c = 0; c < YW; c++) on[c] = true;
            } else if (one_hc[ry]) {
              const bool m = mrow[hc_l[ry][0]] != 0;
#pragma unroll
              for (int c = 0; c < YW; c++) on[c] = m;
            } else {
#pragma unroll
              for (int c = 0; c < YW; c++) on[c] = (col + c < a.M) ? mrow[hc_l[ry][c]] != 0 : false;
            }
#pragma unroll
            for (int c = 0; c < YW; c++) {
              T t = acc[rx * XW + r][ry * YW + c][v] * a.invB;
              t = t * a.tau;
              T cn = cv[c] * a.omt + t;
              cn = cn > T(0) ? cn : T(0);
              cv[c] = cn;
              const T wgt = weight_from_traces<T>(cn, rci, rcj_l[ry][c], a.cthr4);
              wv[c] = on[c] ? wgt : T(0);
            }
            store_w<T, YW, VEC>(cv, crow, col, a.M);
            store_w<T, YW, VEC>(wv, wrow, col, a.M);
          }
        }
      }
}

}  // namespace sb
