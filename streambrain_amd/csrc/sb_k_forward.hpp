// Forward pass: act = softmax_per_hypercolumn(x . W + bias)        omp.cc:70-87 + kernels_numpy.py:13-25
// ("omp.cc" = BCPNN/backend/_kernels/kernels_openmp_internal.cc of the reference)
//
// A workgroup of NWAVES wavefronts owns 16 batch rows x one column tile: one whole hypercolumn when
// FUSE (so the softmax can run in the epilogue), NG*16*VW arbitrary columns otherwise.  The wavefronts
// split the reduction dimension N in interleaved chunks of 4*VW; each runs 16x16x4 MFMAs with
//   A = x : lane (p,q) loads VW consecutive k of batch row b0+p          -> VW MFMA steps
//   B = W : lane (p,q) loads VW consecutive columns of W row k           -> VW column blocks
// so one 16-byte load of x and VW*NG 16-byte loads of W feed VW*VW*NG MFMAs.  Column block c of group
// g holds columns j0 + g*16*VW + VW*p + c (interleaved), which makes every result vector
// {c = 0..VW-1} VW consecutive columns.  Partial tiles are summed through LDS in a fixed tree order,
// then 16 threads per batch row add the bias and, when FUSE, do the softmax.
//
// Tile order: workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.  The kernel
// renumbers them so that one XCD gets a contiguous run of tiles, batch tiles of the same column tile
// adjacent: the W columns of a hypercolumn are then fetched from HBM by one XCD only and shared by
// its workgroups through that XCD's L2.
#pragma once
#include "sb_common.hpp"

namespace sb {

template <typename T>
struct ForwardArgs {
  T *act;
  const T *x;
  const T *W;
  const T *bias;
  long B, N, M, Mc;
  long col_tiles, batch_tiles;
  int dbg;  // profiling experiments: bit0 skip the K loop, bit1 leave before the epilogue
};

// Unguarded 16-byte loads of the main loop: rows / columns outside the matrix are redirected to a valid
// address (their products land in accumulator rows / columns that are never stored), so the loop body
// is loads + MFMAs + pointer bumps only.  The last, partial K chunk takes the guarded path.
template <typename T, int NG, bool FUSE, bool VEC, int NWAVES>
__global__ __launch_bounds__(64 * NWAVES) void k_forward(ForwardArgs<T> a) {
  constexpr int VW = Real<T>::VW;
  constexpr int GW = 16 * VW;
  constexpr int CP = NG * GW + VW;
  constexpr int KC = 4 * VW;  // k per chunk
  using acc_t = typename Real<T>::acc_t;
  using vec_t = typename Real<T>::vec_t;
  __shared__ __attribute__((aligned(16))) T red[NWAVES / 2][16][CP];

  // XCD-aware renumbering (see header comment)
  const long ntiles = a.col_tiles * a.batch_tiles;
  const long per_xcd = (ntiles + 7) / 8;
  const long tile = (long)(blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (tile >= ntiles) return;  // whole workgroup, before any barrier
  const long ct = tile / a.batch_tiles, bt = tile % a.batch_tiles;

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, p = lane & 15, q = lane >> 4;
  const long b0 = bt * 16;
  const long j0 = FUSE ? ct * a.Mc : ct * (NG * GW);
  const long jend = FUSE ? j0 + a.Mc : (j0 + NG * GW < a.M ? j0 + NG * GW : a.M);
  const bool row_ok = (b0 + p) < a.B;
  const T *xrow = a.x + (b0 + p) * a.N;

  acc_t acc[NG][VW];
#pragma unroll
  for (int g = 0; g < NG; g++)
#pragma unroll
    for (int c = 0; c < VW; c++) acc[g][c] = acc_t{0, 0, 0, 0};

  T xa[VW], xb[VW];
  T wa[VW][NG][VW], wb[VW][NG][VW];

  auto compute = [&](const T(&xi)[VW], const T(&wi)[VW][NG][VW]) {
#pragma unroll
    for (int s = 0; s < VW; s++)
#pragma unroll
      for (int g = 0; g < NG; g++)
#pragma unroll
        for (int c = 0; c < VW; c++) acc[g][c] = Real<T>::mfma(xi[s], wi[s][g][c], acc[g][c]);
  };
  auto load_guarded = [&](long kc, T(&xo)[VW], T(&wo)[VW][NG][VW]) {
    const long kk = kc * KC + VW * q;
    load_vw<T, VEC>(xo, xrow, kk, a.N, row_ok);
#pragma unroll
    for (int s = 0; s < VW; s++) {
      const long krow = kk + s;
      const T *wrow = a.W + krow * a.M;
#pragma unroll
      for (int g = 0; g < NG; g++)
        load_vw<T, VEC>(wo[s][g], wrow, j0 + g * GW + VW * p, jend, krow < a.N);
    }
  };

  const long nfull = a.N / KC;  // chunks with all KC reduction indices inside the matrix
  if (a.dbg & 1) {
  } else if (VEC) {
    // per-lane pointers of chunk `w`; every later chunk of this wavefront is NWAVES chunks further on
    const long rowc = row_ok ? b0 + p : a.B - 1;
    const T *xp = a.x + rowc * a.N + (long)w * KC + VW * q;
    const T *wp[VW][NG];
#pragma unroll
    for (int s = 0; s < VW; s++)
#pragma unroll
      for (int g = 0; g < NG; g++) {
        long col = j0 + g * GW + VW * p;
        if (col >= jend) col = j0;  // redirected: feeds unused columns only
        wp[s][g] = a.W + ((long)w * KC + VW * q + s) * a.M + col;
      }
    const long xstep = (long)NWAVES * KC;
    const long wstep = (long)NWAVES * KC * a.M;
    auto load_fast = [&](T(&xo)[VW], T(&wo)[VW][NG][VW]) {
      const vec_t xv = *reinterpret_cast<const vec_t *>(xp);
#pragma unroll
      for (int e = 0; e < VW; e++) xo[e] = xv[e];
      xp += xstep;
#pragma unroll
      for (int s = 0; s < VW; s++)
#pragma unroll
        for (int g = 0; g < NG; g++) {
          const vec_t wv = *reinterpret_cast<const vec_t *>(wp[s][g]);
#pragma unroll
          for (int e = 0; e < VW; e++) wo[s][g][e] = wv[e];
          wp[s][g] += wstep;
        }
    };
    // chunks w, w + NWAVES, ... < nfull, two per iteration with one chunk of loads in flight
    long kc = w;
    if (kc < nfull) load_fast(xa, wa);
    while (kc < nfull) {
      const bool more1 = kc + NWAVES < nfull;
      if (more1) load_fast(xb, wb);
      compute(xa, wa);
      if (!more1) break;
      const bool more2 = kc + 2 * NWAVES < nfull;
      if (more2) load_fast(xa, wa);
      compute(xb, wb);
      if (!more2) break;
      kc += 2 * NWAVES;
    }
    // partial last chunk (N % KC != 0): one wavefront takes it through the guarded path
    if (nfull * KC < a.N && w == (int)(nfull % NWAVES)) {
      load_guarded(nfull, xa, wa);
      compute(xa, wa);
    }
  } else {
    const long nchunks = (a.N + KC - 1) / KC;
    for (long kc = w; kc < nchunks; kc += NWAVES) {
      load_guarded(kc, xa, wa);
      compute(xa, wa);
    }
  }

  if (a.dbg & 2) {
    if (acc[0][0][0] == T(12345.678)) a.act[0] = acc[0][0][0];
    return;
  }
  // ---- cross-wavefront sum through LDS, halving the number of live partials each round:
  //      wavefront w + half stores, wavefront w < half adds.  Fixed order => deterministic.
#pragma unroll
  for (int half = NWAVES / 2; half >= 1; half >>= 1) {
    if (w >= half && w < 2 * half) {
#pragma unroll
      for (int g = 0; g < NG; g++)
#pragma unroll
        for (int v = 0; v < 4; v++) {
          vec_t t;
#pragma unroll
          for (int c = 0; c < VW; c++) t[c] = acc[g][c][v];
          *reinterpret_cast<vec_t *>(&red[w - half][Real<T>::acc_row(q, v)][g * GW + VW * p]) = t;
        }
    }
    __syncthreads();
    if (w < half) {
#pragma unroll
      for (int g = 0; g < NG; g++)
#pragma unroll
        for (int v = 0; v < 4; v++) {
          const vec_t t =
              *reinterpret_cast<const vec_t *>(&red[w][Real<T>::acc_row(q, v)][g * GW + VW * p]);
#pragma unroll
          for (int c = 0; c < VW; c++) acc[g][c][v] += t[c];
        }
    }
    __syncthreads();
  }
  // wavefront 0 now holds the complete tile; publish it for the row-wise epilogue
  if (w == 0) {
#pragma unroll
    for (int g = 0; g < NG; g++)
#pragma unroll
      for (int v = 0; v < 4; v++) {
        vec_t t;
#pragma unroll
        for (int c = 0; c < VW; c++) t[c] = acc[g][c][v];
        *reinterpret_cast<vec_t *>(&red[0][Real<T>::acc_row(q, v)][g * GW + VW * p]) = t;
      }
  }
  __syncthreads();

  // ---- bias (+ softmax): 16 threads per batch row (256 threads), thread handles columns l16 + 16 t
  if (tid >= 256) return;
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
      vals[t] = red[0][row][col] + a.bias[j0 + col];
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

}  // namespace sb
