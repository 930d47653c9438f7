// Forward pass, split-K form: act = softmax_per_hypercolumn(x . W + bias)
//                                                        omp.cc:70-87 + kernels_numpy.py:13-25
// ("omp.cc" = BCPNN/backend/_kernels/kernels_openmp_internal.cc of the reference)
//
// With a small batch the forward GEMM is short and wide (B x M outputs, reduction over N): tiling the
// outputs alone either leaves CUs idle or makes every workgroup re-read its W columns from L2 once per
// 16 batch rows, and L2 bandwidth becomes the bound.  Here a workgroup owns ALL batch rows of a group of
// 128, ONE hypercolumn and ONE slice of the reduction dimension, so every element of W is fetched from
// L2 exactly once per row group:
//   k_forward_splitk   grid = row groups x H x KS.  8 wavefronts, 16 batch rows each.  Per chunk of
//                      4*VW reduction indices the workgroup copies the W chunk [4*VW, hypercolumn] into
//                      LDS (one 16-byte load per thread, double-buffered, one barrier per chunk); each
//                      wavefront loads its own x operand straight from global memory (lane (p,q): VW
//                      consecutive k of batch row p, feeding VW MFMA steps) and reads W from LDS as
//                      16-byte vectors (VW column blocks per read, columns interleaved exactly as in
//                      k_forward).  The partial tile goes to part[ks][b][j].
//   k_forward_finish   one wavefront per (batch row, hypercolumn): sums the KS partials in slice order,
//                      adds the bias, applies the softmax, writes act.
#pragma once
#include <type_traits>

#include "sb_common.hpp"

// Hook for phase timing in development builds; expands to nothing in the library.
#ifndef SB_PHASE_MARK
#define SB_PHASE_MARK(n)
#endif

namespace sb {

template <typename T>
struct ForwardSplitArgs {
  T *part;  // [KS, B, M]
  const T *x;
  const T *W;
  long B, N, M, H, Mc;
  long KS;            // slices of the reduction dimension
  long chunks_total;  // ceil(N / (4*VW))
  int dbg;            // profiling experiments: bit0 skip the chunk loop, bit1 skip the partial stores
};

template <typename T, int NG, bool VEC>
__global__ __launch_bounds__(512) void k_forward_splitk(ForwardSplitArgs<T> a) {
  using R = Real<T>;
  using acc_t = typename R::acc_t;
  using vec_t = typename R::vec_t;
  constexpr int VW = R::VW;
  constexpr int GW = 16 * VW;
  constexpr int KC = 4 * VW;              // reduction indices per chunk
  constexpr int CW = NG * GW;             // staged columns (hypercolumn, padded)
  constexpr int NV = KC * CW / VW;        // 16-byte vectors per staged chunk
  constexpr int PER = (NV + 511) / 512;   // vectors per thread
  __shared__ __attribute__((aligned(16))) T ws[4][KC][CW];  // ring of 4 staged chunks

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, p = lane & 15, q = lane >> 4;
  const long ks = (long)blockIdx.x % a.KS;
  const long h = ((long)blockIdx.x / a.KS) % a.H;
  const long rg = (long)blockIdx.x / (a.KS * a.H);
  const long c0 = ks * a.chunks_total / a.KS, c1 = (ks + 1) * a.chunks_total / a.KS;
  const long j0 = h * a.Mc;
  const long b0 = rg * 128 + 16 * w;
  const bool row_ok = b0 + p < a.B;
  const T *xrow = a.x + (row_ok ? b0 + p : a.B - 1) * a.N;  // rows past the batch read a valid row

  acc_t acc[NG][VW];
#pragma unroll
  for (int g = 0; g < NG; g++)
#pragma unroll
    for (int c = 0; c < VW; c++) acc[g][c] = acc_t{0, 0, 0, 0};

  // Register ring of PF chunks in flight (W share + x operand: 2 vectors per thread and chunk), LDS ring
  // of 2: chunk c is computed from LDS while chunk c+1 moves registers -> LDS and chunk c+PF is requested.
  constexpr int PF = 4;
  T wreg[PF][PER][VW], xreg[PF][VW];
  auto load_chunk = [&](long chunk, T(&wo)[PER][VW], T(&xo)[VW]) {
    const bool live = chunk < c1;
#pragma unroll
    for (int u = 0; u < PER; u++) {
      const int v = tid + 512 * u;
      const int kr = v / (CW / VW), cv = v % (CW / VW);
      const long k = chunk * KC + kr;
      if (VEC)
        load_vw_sel<T>(wo[u], a.W + k * a.M + j0 + VW * cv, a.W,
                       live && v < NV && k < a.N && VW * cv < a.Mc);
      else
        load_vw<T, false>(wo[u], a.W + k * a.M + j0, (long)VW * cv, a.Mc, live && v < NV && k < a.N);
    }
    const long kk = chunk * KC + VW * q;
    if (VEC)
      load_vw_sel<T>(xo, xrow + kk, a.x, live && kk < a.N);
    else
      load_vw<T, false>(xo, xrow, kk, a.N, live);
  };
  auto store_w_chunk = [&](int buf, const T(&wi)[PER][VW]) {
#pragma unroll
    for (int u = 0; u < PER; u++) {
      const int v = tid + 512 * u;
      if (v < NV) {
        vec_t t;
#pragma unroll
        for (int e = 0; e < VW; e++) t[e] = wi[u][e];
        *reinterpret_cast<vec_t *>(&ws[buf][v / (CW / VW)][VW * (v % (CW / VW))]) = t;
      }
    }
  };

  // Three-stage pipeline, one barrier per chunk.  At the step of chunk cc:
  //   MFMAs run on registers wv[cc&1] (read from LDS during the previous step),
  //   the LDS reads of chunk cc+1 are issued into wv[(cc+1)&1],
  //   chunk cc+2 moves from the register ring to its LDS slot, chunk cc+PF is requested from L2.
  // No branches inside (loads are select-guarded; chunks past the slice are zeros nobody uses), so wait
  // counts stay exact and the loads really are in flight across steps.
  vec_t wvA[VW][NG], wvB[VW][NG];
  auto read_lds = [&](int slot, vec_t(&wv)[VW][NG]) {
#pragma unroll
    for (int s = 0; s < VW; s++)
#pragma unroll
      for (int g = 0; g < NG; g++)
        wv[s][g] = *reinterpret_cast<const vec_t *>(&ws[slot][VW * q + s][g * GW + VW * p]);
  };
  auto mfmas = [&](const T(&xa)[VW], const vec_t(&wv)[VW][NG]) {
#pragma unroll
    for (int s = 0; s < VW; s++)
#pragma unroll
      for (int g = 0; g < NG; g++)
#pragma unroll
        for (int k2 = 0; k2 < VW; k2++) acc[g][k2] = R::mfma(xa[s], wv[s][g][k2], acc[g][k2]);
  };
  auto step = [&](auto U, long cc) {
    constexpr int u = decltype(U)::value;
    T xa[VW];
#pragma unroll
    for (int e = 0; e < VW; e++) xa[e] = xreg[u][e];
    if (u & 1) {
      read_lds((u + 1) % PF, wvA);
      mfmas(xa, wvB);
    } else {
      read_lds((u + 1) % PF, wvB);
      mfmas(xa, wvA);
    }
    store_w_chunk((u + 2) % PF, wreg[(u + 2) % PF]);
    load_chunk(cc + PF, wreg[u], xreg[u]);
    __syncthreads();
  };
#pragma unroll
  for (int u = 0; u < PF; u++) load_chunk(c0 + u, wreg[u], xreg[u]);
  SB_PHASE_MARK(0);
  store_w_chunk(0, wreg[0]);
  store_w_chunk(1, wreg[1]);
  __syncthreads();
  SB_PHASE_MARK(2);
  read_lds(0, wvA);
  long c = (a.dbg & 1) ? c1 : c0;
  for (; c + PF <= c1; c += PF) {
    step(std::integral_constant<int, 0>{}, c);
    step(std::integral_constant<int, 1>{}, c + 1);
    step(std::integral_constant<int, 2>{}, c + 2);
    step(std::integral_constant<int, 3>{}, c + 3);
  }
  static_assert(PF == 4, "the unrolled steps above and below assume rings of 4");
  if (c < c1) step(std::integral_constant<int, 0>{}, c);
  if (c + 1 < c1) step(std::integral_constant<int, 1>{}, c + 1);
  if (c + 2 < c1) step(std::integral_constant<int, 2>{}, c + 2);

  SB_PHASE_MARK(1);
  if (a.dbg & 2) {
    if (acc[0][0][0] == T(12345.678)) a.part[0] = acc[0][0][0];
    return;
  }
  // partial tile -> part[ks][b][j]
#pragma unroll
  for (int g = 0; g < NG; g++)
#pragma unroll
    for (int v = 0; v < 4; v++) {
      const long brow = b0 + R::acc_row(q, v);
      if (brow < a.B) {
        T t[VW];
#pragma unroll
        for (int cc = 0; cc < VW; cc++) t[cc] = acc[g][cc][v];
        store_vw<T, VEC>(t, a.part + (ks * a.B + brow) * a.M + j0, (long)g * GW + VW * p, a.Mc);
      }
    }
  SB_PHASE_MARK(3);
}

// One wavefront per (batch row, hypercolumn).
template <typename T>
__global__ __launch_bounds__(256) void k_forward_finish(T *act, const T *part, const T *bias, long B,
                                                        long M, long H, long Mc, long KS, int softmax) {
  const int lane = threadIdx.x & 63;
  const long g = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (g >= B * H) return;
  const long b = g / H, h = g % H;
  T *out = act + b * M + h * Mc;
  const T *src = part + b * M + h * Mc;
  const T *bs = bias + h * Mc;
  const long stride = B * M;
  T mx = -INFINITY;
  for (long c = lane; c < Mc; c += 64) {
    T s = T(0);
    for (long k0 = 0; k0 < KS; k0 += 8) {  // 8 slices in flight, added in slice order
      T v[8];
#pragma unroll
      for (int k = 0; k < 8; k++) v[k] = (k0 + k < KS) ? src[(k0 + k) * stride + c] : T(0);
#pragma unroll
      for (int k = 0; k < 8; k++) s += v[k];
    }
    s += bs[c];
    out[c] = s;
    mx = s > mx ? s : mx;
  }
  if (!softmax) return;
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    const T other = __shfl_xor(mx, o);
    mx = other > mx ? other : mx;
  }
  T sum = T(0);
  for (long c = lane; c < Mc; c += 64) {  // each lane re-reads only what it wrote itself
    const T e = Real<T>::exp_(out[c] - mx);
    out[c] = e;
    sum += e;
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) sum += __shfl_xor(sum, o);
  for (long c = lane; c < Mc; c += 64) out[c] = out[c] / sum;
}

}  // namespace sb
