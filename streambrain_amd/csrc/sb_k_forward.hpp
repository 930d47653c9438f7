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
// {c = 0..VW-1} VW consecutive columns.  Partial tiles are summed through LDS in a fixed order, then
// 16 threads per batch row add the bias and, when FUSE, do the softmax.
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
  FastDiv by_batch_tiles;  // division by batch_tiles (set by the launcher along with it)
};

// Column layout of a tile, shared by the kernels below: NG groups of 16 lanes-columns, group g holding
// VW column blocks (the last group LW <= VW), lane p of a group owning gwidth(g) consecutive columns.
template <typename T, int NG, int LW>
struct TileCols {
  static constexpr int VW = Real<T>::VW;
  static constexpr int GW = 16 * VW;
  static constexpr int CP = NG * GW + VW;  // padded row length of a tile in LDS
  __device__ static constexpr int gwidth(int g) { return g == NG - 1 ? LW : VW; }
  __device__ static constexpr int gcol(int g, int p) { return g * GW + gwidth(g) * p; }
};

template <typename T, int LW>
struct PackedCols {  // LW consecutive elements, element-aligned
  T v[LW];
} __attribute__((packed, aligned(sizeof(T))));

// The epilogue's split of a tile row over threads: all 64*NWAVES threads take part, TPR of them per batch
// row (a power of two, at most 64, so a row never straddles wavefronts), each with PT columns
// lr + TPR t.  load() fetches the thread's bias values; the kernels call it ahead of their main loop so
// that the latency is not added to the epilogue.
template <typename T, int NG, int NWAVES>
struct ForwardBias {
  static constexpr int TPR = 4 * NWAVES;
  static constexpr int COLS = NG * 16 * Real<T>::VW;
  static constexpr int PT = (COLS + TPR - 1) / TPR;
  static_assert(TPR <= 64, "a batch row's threads must lie in one wavefront");
  __device__ static __forceinline__ void load(T (&bv)[PT], const T *bias, long j0, long ncol) {
    const int lr = threadIdx.x % TPR;
#pragma unroll
    for (int t = 0; t < PT; t++) {
      const long col = lr + TPR * t;
      bv[t] = bias[j0 + (col < ncol ? col : 0)];
    }
  }
};

// Tail of the forward kernels: the NWAVES partial tiles (one per wavefront, in MFMA accumulator layout)
// are summed through LDS in a fixed order (deterministic), then 16 threads per batch row add the bias
// and, when FUSE, do the softmax over the tile's ncol columns.  bv: the thread's bias values
// (ForwardBias::load).
// tail: with TAIL, the tile's last four columns (tail_col0 .. +3 of the tile) as the 4x4 products of
// Real<T>::mfma_4x4 leave them: element v of lane (p, q) is row 4 (p/4) + v, column p % 4, summed over the
// reduction indices of q only.
// NT: tiles of LDS the partial sums go through.  NWAVES / 2: the two-step hand-over described below.  NWAVES: every
// wavefront puts its partial tile down and the row-wise pass adds up all of them -- twice the LDS, one barrier
// and one dependent round trip through LDS less (for the kernels whose time is a chain of latencies).
template <typename T, int NG, bool FUSE, int NWAVES, int LW, bool TAIL = false, int NT = NWAVES / 2>
__device__ __forceinline__ void forward_finish(const typename Real<T>::acc_t (&acc)[NG][Real<T>::VW],
                                               const T (&bv)[ForwardBias<T, NG, NWAVES>::PT],
                                               T (&red)[NT][16][TileCols<T, NG, LW>::CP], T *act,
                                               long B, long M, long b0, long j0, long ncol,
                                               typename Real<T>::acc_t tail = {}) {
  static_assert(NT == NWAVES / 2 || NT == NWAVES, "tiles of partial sums");
  using TC = TileCols<T, NG, LW>;
  constexpr int VW = Real<T>::VW;
  using vec_t = typename Real<T>::vec_t;
  auto gwidth = [](int g) { return TC::gwidth(g); };
  auto gcol = [](int g, int p_) { return TC::gcol(g, p_); };
  const int tid = threadIdx.x, lane = tid & 63, p = lane & 15, q = lane >> 4;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr int tail_col0 = (NG - 1) * TC::GW + 16 * LW;
  if constexpr (TAIL) {
    static_assert(tail_col0 + 4 <= TC::CP, "tail columns inside the padded LDS row");
#pragma unroll
    for (int v = 0; v < 4; v++) {  // the four q in a fixed order
      tail[v] += __shfl_xor(tail[v], 16);
      tail[v] += __shfl_xor(tail[v], 32);
    }
  }
  // ---- cross-wavefront sum through LDS in a fixed order (deterministic): the upper half of the
  // wavefronts hands its partial tiles over, the lower half adds them to its own and publishes the
  // sums (each lane rewrites exactly the elements it has just read, so no barrier is needed between
  // the two); the row-wise epilogue then adds up the HALF published tiles.
  constexpr int HALF = NWAVES / 2;
  static_assert(NWAVES >= 2 && (NWAVES & (NWAVES - 1)) == 0, "a power of two, at least 2 wavefronts");
  if constexpr (NT == NWAVES) {
#pragma unroll
    for (int g = 0; g < NG; g++)
#pragma unroll
      for (int v = 0; v < 4; v++) {
        T *slot = &red[w][Real<T>::acc_row(q, v)][gcol(g, p)];
        if (gwidth(g) == VW) {
          vec_t t;
#pragma unroll
          for (int c = 0; c < VW; c++) t[c] = acc[g][c][v];
          *reinterpret_cast<vec_t *>(slot) = t;
        } else {
#pragma unroll
          for (int c = 0; c < LW; c++) slot[c] = acc[g][c][v];
        }
      }
    if (TAIL && q == 0) {
#pragma unroll
      for (int v = 0; v < 4; v++) red[w][4 * (p >> 2) + v][tail_col0 + (p & 3)] = tail[v];
    }
  } else {
  if (w >= HALF) {
#pragma unroll
    for (int g = 0; g < NG; g++)
#pragma unroll
      for (int v = 0; v < 4; v++) {
        T *slot = &red[w - HALF][Real<T>::acc_row(q, v)][gcol(g, p)];
        if (gwidth(g) == VW) {
          vec_t t;
#pragma unroll
          for (int c = 0; c < VW; c++) t[c] = acc[g][c][v];
          *reinterpret_cast<vec_t *>(slot) = t;
        } else {
#pragma unroll
          for (int c = 0; c < LW; c++) slot[c] = acc[g][c][v];
        }
      }
    if (TAIL && q == 0) {
#pragma unroll
      for (int v = 0; v < 4; v++) red[w - HALF][4 * (p >> 2) + v][tail_col0 + (p & 3)] = tail[v];
    }
  }
  __syncthreads();
  if (w < HALF) {
#pragma unroll
    for (int g = 0; g < NG; g++)
#pragma unroll
      for (int v = 0; v < 4; v++) {
        T *slot = &red[w][Real<T>::acc_row(q, v)][gcol(g, p)];
        if (gwidth(g) == VW) {
          vec_t t = *reinterpret_cast<vec_t *>(slot);
#pragma unroll
          for (int c = 0; c < VW; c++) t[c] += acc[g][c][v];
          *reinterpret_cast<vec_t *>(slot) = t;
        } else {
#pragma unroll
          for (int c = 0; c < LW; c++) slot[c] += acc[g][c][v];
        }
      }
    if (TAIL && q == 0) {
#pragma unroll
      for (int v = 0; v < 4; v++) red[w][4 * (p >> 2) + v][tail_col0 + (p & 3)] += tail[v];
    }
  }
  }
  __syncthreads();
  // ---- bias (+ softmax): TPR threads per batch row, thread handles columns lr + TPR t
  constexpr int TPR = ForwardBias<T, NG, NWAVES>::TPR, PT = ForwardBias<T, NG, NWAVES>::PT;
  const int row = tid / TPR, lr = tid % TPR;
  T vals[PT];
  T mx = -INFINITY;
#pragma unroll
  for (int t = 0; t < PT; t++) {
    const long col = lr + TPR * t;
    T sum = red[0][row][col < ncol ? col : 0];
#pragma unroll
    for (int h = 1; h < NT; h++) sum += red[h][row][col < ncol ? col : 0];
    vals[t] = col < ncol ? sum + bv[t] : T(0);
    mx = (col < ncol && vals[t] > mx) ? vals[t] : mx;
  }
  if (FUSE) {
    // across the TPR threads of the batch row: rows of 16 lanes by DPP moves, then across rows
    static_assert(TPR >= 16, "at least one row of 16 lanes per batch row");
    mx = row16_reduce(mx, [](T x_, T y_) { return y_ > x_ ? y_ : x_; });
#pragma unroll
    for (int o = TPR / 2; o >= 16; o >>= 1) {
      const T other = __shfl_xor(mx, o);
      mx = other > mx ? other : mx;
    }
    T sum = T(0);
#pragma unroll
    for (int t = 0; t < PT; t++) {
      const long col = lr + TPR * t;
      if (col < ncol) {
        vals[t] = Real<T>::exp_nonpos(vals[t] - mx);
        sum += vals[t];
      }
    }
    sum = row16_reduce(sum, [](T x_, T y_) { return x_ + y_; });
#pragma unroll
    for (int o = TPR / 2; o >= 16; o >>= 1) sum += __shfl_xor(sum, o);
    if constexpr (sizeof(T) == 4) {  // one division per row, then products
      const T r = T(1) / sum;
#pragma unroll
      for (int t = 0; t < PT; t++) vals[t] = vals[t] * r;
    } else {
#pragma unroll
      for (int t = 0; t < PT; t++) vals[t] = vals[t] / sum;
    }
  }
  if (b0 + row < B) {
    T *out = act + (b0 + row) * M + j0;
#pragma unroll
    for (int t = 0; t < PT; t++) {
      const long col = lr + TPR * t;
      if (col < ncol) out[col] = vals[t];
    }
  }
}

// Main loop: x and W are read with 16-byte loads through bounds-checked buffer windows, so rows and
// columns outside the matrices read zero and the loop body is loads + MFMAs only.  Without VEC (shapes
// without 16-byte alignment) the same loads start at any element -- multi-dword accesses need dword
// alignment only -- and a vector that straddles the end of the tile also fetches a few columns of the
// neighbouring tile, which land in accumulator columns the epilogue never reads (at the very end of W the
// window's range check, which is per dword, returns zeros for them).  The last, partial K chunk takes the
// guarded path.
// One workgroup per CU is all the tiling provides at small batch sizes, so the register allocator is told
// to aim for NWAVES/4 wavefronts per SIMD and spend the registers on loads in flight instead.
//
// LW: column blocks of the LAST group (1..VW).  A hypercolumn of 100 columns needs 7 blocks of 16, not
// 8: with LW = 3 the last group's lanes load LW consecutive columns (12 bytes) instead of VW, and a
// quarter of that group's MFMAs disappears.  The launcher picks LW < VW only when no vector of the last
// group straddles the end of the tile.
//
// RB: row blocks per workgroup.  The tile is 16*RB batch rows, every W vector a lane loads feeds RB MFMAs
// instead of one, and W crosses the L2 -> L1 path 1/RB as often: for batches of many rows, where that path
// is what bounds the kernel.  The epilogue handles the row blocks one after the other.
//
// TAIL (float): the hypercolumn ends with four columns beyond the last group's blocks (100 = 6 blocks of 16
// + 4).  Instead of a seventh block, three quarters of it padding, they are multiplied as 4x4 products
// (Real<T>::mfma_4x4) that take the x operand registers of the 16x16x4 form as they are and one extra
// element of W per lane and step, at a quarter of a block's cost.
template <typename T, int NG, bool FUSE, bool VEC, int NWAVES, int LW = Real<T>::VW, int RB = 1, bool TAIL = false>
__global__ __launch_bounds__(64 * NWAVES) __attribute__((amdgpu_waves_per_eu(NWAVES / 4, NWAVES / 4)))
void k_forward(ForwardArgs<T> a) {
  constexpr int VW = Real<T>::VW;
  static_assert(LW >= 1 && LW <= VW, "width of the last group");
  static_assert(!TAIL || (sizeof(T) == 4 && FUSE && VEC), "the four-column tail: float, fused, vector loads");
  constexpr int tail_col0 = (NG - 1) * 16 * VW + 16 * LW;  // first tail column of the tile
  auto gwidth = [](int g) { return g == NG - 1 ? LW : VW; };         // column blocks of group g
  auto gcol = [&](int g, int p_) { return g * (16 * VW) + gwidth(g) * p_; };  // first tile column of lane p_
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
  const long ct = a.by_batch_tiles.div((uint32_t)tile), bt = tile - ct * a.batch_tiles;  // tile < 2^31

  const int tid = threadIdx.x, lane = tid & 63, p = lane & 15, q = lane >> 4;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave index, in a scalar register: uniform branches
  const long b0 = bt * (16 * RB);
  const long j0 = FUSE ? ct * a.Mc : ct * (NG * GW);
  const long jend = FUSE ? j0 + a.Mc : (j0 + NG * GW < a.M ? j0 + NG * GW : a.M);

  acc_t acc[RB][NG][VW];
#pragma unroll
  for (int r = 0; r < RB; r++)
#pragma unroll
    for (int g = 0; g < NG; g++)
#pragma unroll
      for (int c = 0; c < VW; c++) acc[r][g][c] = acc_t{0, 0, 0, 0};
  acc_t tacc[RB];
#pragma unroll
  for (int r = 0; r < RB; r++) tacc[r] = acc_t{0, 0, 0, 0};

  // ring of D chunk buffers: D-1 chunks of loads are in flight while one is being multiplied
  constexpr int D = 2;  // measured: deeper rings are slower, the CU cannot keep more loads in flight anyway
  T xr[D][RB][VW];
  T wr[D][VW][NG][VW];
  T wt[D][VW];  // TAIL: W[k, tail column p % 4] for the lane's VW reduction indices

  auto compute = [&](const T(&xi)[RB][VW], const T(&wi)[VW][NG][VW], const T(&ti)[VW]) {
#pragma unroll
    for (int s = 0; s < VW; s++) {
#pragma unroll
      for (int g = 0; g < NG; g++)
#pragma unroll
        for (int c = 0; c < VW; c++)
          if (c < gwidth(g)) {
#pragma unroll
            for (int r = 0; r < RB; r++) acc[r][g][c] = Real<T>::mfma(xi[r][s], wi[s][g][c], acc[r][g][c]);
          }
      if constexpr (TAIL) {
#pragma unroll
        for (int r = 0; r < RB; r++) tacc[r] = Real<T>::mfma_4x4(xi[r][s], ti[s], tacc[r]);
      }
    }
  };
  auto load_guarded = [&](long kc, T(&xo)[RB][VW], T(&wo)[VW][NG][VW], T(&to)[VW]) {
    const long kk = kc * KC + VW * q;
#pragma unroll
    for (int r = 0; r < RB; r++) {
      const long row = b0 + 16 * r + p;
      load_vw<T, VEC>(xo[r], a.x + (row < a.B ? row : 0) * a.N, kk, a.N, row < a.B);
    }
#pragma unroll
    for (int s = 0; s < VW; s++) {
      const long krow = kk + s;
      const T *wrow = a.W + krow * a.M;
#pragma unroll
      for (int g = 0; g < NG; g++) {
        if (gwidth(g) == VW) {
          load_vw<T, VEC>(wo[s][g], wrow, j0 + g * GW + VW * p, jend, krow < a.N);
        } else {
#pragma unroll
          for (int e = 0; e < LW; e++) {
            const long col = j0 + gcol(g, p) + e;
            wo[s][g][e] = (krow < a.N && col < jend) ? wrow[col] : T(0);
          }
        }
      }
      if constexpr (TAIL) to[s] = krow < a.N ? wrow[j0 + tail_col0 + (p & 3)] : T(0);
    }
  };

  // the epilogue's bias values are requested before the K loop, so their latency is not added to it
  const long ncol = jend - j0;
  T bv[ForwardBias<T, NG, NWAVES>::PT];
  ForwardBias<T, NG, NWAVES>::load(bv, a.bias, j0, ncol);
  const long nfull = a.N / KC;  // chunks with all KC reduction indices inside the matrix
  {
    // Chunk `w` first; every later chunk of this wavefront is NWAVES chunks further on.  x and W are
    // reached through bounds-checked buffer windows that start at the chunk (a scalar base address,
    // advanced with scalar instructions), so the per-lane offsets never change and the loop body is
    // loads and MFMAs only.  Batch rows past the end and columns past the tile read zero.
    constexpr unsigned ES = sizeof(T);
    const T *xbase = a.x + b0 * a.N + (long)w * KC;             // uniform
    const T *wbase = a.W + (long)w * KC * a.M + j0;             // uniform
    long xleft = (a.B - b0) * a.N - (long)w * KC;               // elements from xbase to the end of x
    long wleft = (a.N - (long)w * KC) * a.M - j0;               // ... of W
    unsigned xat[RB];
#pragma unroll
    for (int r = 0; r < RB; r++) xat[r] = (unsigned)(((long)(16 * r + p) * a.N + VW * q) * ES);
    unsigned wat[VW][NG];
#pragma unroll
    for (int s = 0; s < VW; s++)
#pragma unroll
      for (int g = 0; g < NG; g++)
        wat[s][g] = j0 + gcol(g, p) < jend ? (unsigned)(((long)(VW * q + s) * a.M + gcol(g, p)) * ES)
                                           : BufferWindow<T>::kOutside;
    unsigned tat[VW];  // TAIL
#pragma unroll
    for (int s = 0; s < VW; s++) tat[s] = (unsigned)(((long)(VW * q + s) * a.M + tail_col0 + (p & 3)) * ES);
    const long xstep = (long)NWAVES * KC;
    const long wstep = (long)NWAVES * KC * a.M;
    // Chunks w, w + NWAVES, ... < nfull: n of them for this wavefront.  The loop is branch-free: a load
    // past the last chunk reads whatever lies there (or zeros past the arrays) and is never used, so
    // the compiler can keep exact wait counts and D-1 chunks really are in flight.
    const long n = w < nfull ? (nfull - 1 - w) / NWAVES + 1 : 0;
    auto load_next = [&](T(&xo)[RB][VW], T(&wo)[VW][NG][VW], T(&to)[VW]) {
      const BufferWindow<T> xwin(xbase, xleft), wwin(wbase, wleft);
#pragma unroll
      for (int r = 0; r < RB; r++) xwin.template load_n<VW>(xo[r], xat[r]);
#pragma unroll
      for (int s = 0; s < VW; s++) {
        if constexpr (TAIL) {
          T one[1];
          wwin.template load_n<1>(one, tat[s]);
          to[s] = one[0];
        }
#pragma unroll
        for (int g = 0; g < NG; g++) {
          if (gwidth(g) == VW) {
            wwin.template load_n<VW>(wo[s][g], wat[s][g]);
          } else {
            T t[LW];
            wwin.template load_n<LW>(t, wat[s][g]);
#pragma unroll
            for (int e = 0; e < LW; e++) wo[s][g][e] = t[e];
          }
        }
      }
      xbase += xstep, xleft -= xstep;
      wbase += wstep, wleft -= wstep;
    };
    if (n > 0) {
#pragma unroll
      for (int u = 0; u < D - 1; u++) load_next(xr[u], wr[u], wt[u]);  // chunks 0 .. D-2
      __builtin_amdgcn_sched_barrier(0);
      long i = 0;
      for (; i + D <= n; i += D) {
#pragma unroll
        for (int u = 0; u < D; u++) {
          // the scheduling fences keep the loads where they are written: the compiler's latency model
          // would otherwise sink them to just ahead of their use, far too late for HBM or L2
          load_next(xr[(u + D - 1) % D], wr[(u + D - 1) % D], wt[(u + D - 1) % D]);  // chunk i + u + D - 1
          __builtin_amdgcn_sched_barrier(0);
          compute(xr[u], wr[u], wt[u]);                                       // chunk i + u
          __builtin_amdgcn_sched_barrier(0);
        }
      }
#pragma unroll
      for (int u = 0; u < D - 1; u++)
        if (i + u < n) compute(xr[u], wr[u], wt[u]);
    }
    // partial last chunk (N % KC != 0): one wavefront takes it through the guarded path
    if (nfull * KC < a.N && w == (int)(nfull % NWAVES)) {
      load_guarded(nfull, xr[0], wr[0], wt[0]);
      compute(xr[0], wr[0], wt[0]);
    }
  }
#pragma unroll
  for (int r = 0; r < RB; r++) {
    if (r > 0) __syncthreads();  // the previous row block's sums have been read
    forward_finish<T, NG, FUSE, NWAVES, LW, TAIL>(acc[r], bv, red, a.act, a.B, a.M, b0 + 16 * r, j0, ncol, tacc[r]);
  }
}

}  // namespace sb
