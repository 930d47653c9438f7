// Fused training pass of one layer: Ci / Cj / Cij moving averages, weight recompute, regularised bias
// and mask apply in ONE kernel.                          omp.cc:89-205 (+ :222-246, :322-335)
// ("omp.cc" = BCPNN/backend/_kernels/kernels_openmp_internal.cc of the reference)
//
//   Ci  <- max(0, Ci*(1-t) + mean_b x[b,i] * t)           Cj likewise from y
//   Cij <- max(0, Cij*(1-t) + (x^T y / B) * t)
//   W   <- wmask ? log(max(Cij, cthr^4) / (Ci*Cj)) : 0     (0 as well where Ci < cthr or Cj < cthr)
//   bias/kbi <- update_bias_regularized(Cj)                (plastic layers)
// all from the NEW traces, as the reference's fused loop does.
//
// A workgroup (256 threads, 4 wavefronts) owns a 64 x 64 tile of Cij; 16 KiB of LDS and at most 96
// registers per thread let five workgroups share a CU, so the 1175 tiles of a 1568 x 3000 layer are
// all resident at once.
//   1. Per chunk of KCH batch rows it stages x[:, i-tile] and y[:, j-tile] in LDS.  x and y are
//      "k-major" in memory, which is the 16x16x4 MFMA operand layout, so staging is a plain copy and
//      each wavefront feeds its 32 x 32 sub-tile (2 x 2 MFMA blocks) with two 8-byte LDS reads per K
//      step of 4.  The global loads of chunk c+1 are issued before chunk c is consumed.
//   2. From the same LDS slabs, the lanes of one wavefront add up one column each of x, those of
//      another one column each of y (which two wavefronts rotates with the tile index), in batch order
//      b = 0..B-1 without FMA contraction: the reference's summation order, so Ci, Cj and kbi stay
//      bit-exact against a strict-IEEE build of it.  Every tile needs Ci for its rows and Cj
//      for its columns, so every workgroup recomputes them from the OLD traces (a tile row shares x,
//      a tile column shares y: same inputs, same order, same bits).  The old traces are read from
//      Ci/Cj and the new ones written to Ci_next/Cj_next by the tiles of the first tile column / row:
//      no workgroup ever reads a value another one is writing.
//   3. Global loads return in issue order, so the Cij tile (HBM latency) is requested only while the
//      second-to-last chunk is being multiplied: the MFMA loop never waits for it, and it has arrived
//      by the time the epilogue needs it.  All loads are branch-free (bounds-checked buffer windows
//      instead of guards): a guarded load makes the compiler wait for every outstanding load at the
//      join.
//   4. The accumulators go through LDS into a row-major layout; each thread then finishes VW consecutive
//      columns of 4 rows: decay + clamp, weight, mask, one 16-byte store each to Cij and W.  With
//      w_masked, a wavefront whose vectors of a pass all lie under zero mask bytes skips the weight.
#pragma once
#include <type_traits>

#include "sb_kernels.hpp"

// Hook for phase timing in development builds; expands to nothing in the library.
#ifndef SB_PHASE_MARK
#define SB_PHASE_MARK(n)
#endif

namespace sb {

template <typename T>
struct TrainArgs {
  const T *x;  // [B,N]
  const T *y;  // [B,M]
  T *Cij;
  T *W;          // nullptr: the traces are updated and no weights are written
  const T *Ci;   // old traces (read)
  const T *Cj;
  T *Ci_next;    // new traces (written by the first tile column / row)
  T *Cj_next;
  const uint8_t *wmask;  // [N,H] or nullptr (no mask: every synapse active)
  int w_masked;          // W is already zero wherever wmask is 0: such entries need not be written
  int bias_mode;         // 0: leave bias alone; 1: update_bias_regularized on the new Cj
  T *bias, *kbi;
  long B, N, M, H, Mc;
  T tau, omt, fB, invB, cthr, cthr4;
  T khalf, pmin, taubdt;
  long tiles_i, tiles_j;
  FastDiv by_panel, by_Mc;  // divisions by tiles_i * panel_cols and by Mc
  unsigned panel_cols;      // tile order: panels of this many tile columns (a power of two), see the kernel
};

// New trace from the old one and the batch's column sum, in the reference's order of operations
// (kernels_openmp_internal.cc:117-129): sum / B, times tau, plus old * (1 - tau), clamped at 0.
template <typename T>
__device__ inline T trace_next(T cold, T sum, const TrainArgs<T> &a) {
  using R = Real<T>;
  T s = R::div(sum, a.fB);
  s = R::mul(s, a.tau);
  const T c = R::add(R::mul(cold, a.omt), s);
  return c > T(0) ? c : T(0);
}

// The new traces Ci_next, Cj_next (and the regularized bias) on their own, a thread per input or output
// unit walking the batch in order: what every tile of k_train_fused otherwise repeats for its own 64 rows
// and 64 columns.  Launched ahead of k_train_fused<.., PRE = true> when a layer has so many tiles that the
// repetition costs more than a launch.
template <typename T>
__global__ __launch_bounds__(256) void k_trace_sums(TrainArgs<T> a) {
  using R = Real<T>;
  const long t = (long)blockIdx.x * 256 + threadIdx.x;
  const bool is_i = t < a.N;
  const long idx = is_i ? t : t - a.N;
  if (!is_i && idx >= a.M) return;
  const T *p = (is_i ? a.x : a.y) + idx;
  const long stride = is_i ? a.N : a.M;
  T sum = T(0);
  long b = 0;
  for (; b + 16 <= a.B; b += 16) {  // 16 loads in flight, then the ordered additions
    T v[16];
#pragma unroll
    for (int k = 0; k < 16; k++) v[k] = p[(b + k) * stride];
#pragma unroll
    for (int k = 0; k < 16; k++) sum = R::add(sum, v[k]);
  }
  for (; b < a.B; b++) sum = R::add(sum, p[b * stride]);
  const T cnew = trace_next<T>((is_i ? a.Ci : a.Cj)[idx], sum, a);
  if (is_i) {
    a.Ci_next[idx] = cnew;
  } else {
    a.Cj_next[idx] = cnew;
    if (a.bias_mode == 1) {
      T kb = a.kbi[idx];
      a.bias[idx] = bias_regularized<T>(cnew, kb, a.cthr, a.khalf, a.pmin, a.taubdt);
      a.kbi[idx] = kb;
    }
  }
}

// Wavefronts per SIMD the registers are budgeted for.  Doubles: four (the LDS slabs allow four workgroups
// per CU; left alone the compiler takes 176 registers, which allows two).  Floats need no limit: 80-96.
template <typename T>
constexpr int train_waves_per_simd() { return sizeof(T) == 8 ? 4 : 1; }
// VEC: Cij and W are stored as 16-byte vectors (M a multiple of VW), element by element otherwise.  Loads
// are 16-byte accesses either way: one that runs over the end of a row of x, y or Cij fetches elements of
// the next row into tile rows / columns outside the matrix, which are never stored or summed.
// MB: mask bytes fetched per vector of VW columns -- 1 when Mc is a multiple of VW (every vector lies
// inside one hypercolumn), VW otherwise.
// PRE: Ci_next and Cj_next already hold the new traces (k_trace_sums): no column sums here.
template <typename T, int KCH, bool VEC, int MB, bool PRE = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(train_waves_per_simd<T>())))
void k_train_fused(TrainArgs<T> a) {
  using R = Real<T>;
  using acc_t = typename R::acc_t;
  constexpr int VW = R::VW;             // elements per 16-byte vector
  constexpr int TS = 64;                // tile side
  constexpr int G = TS / VW;            // 16-byte groups per tile row
  constexpr int RPP = 256 / G;          // tile rows covered by the workgroup per pass
  constexpr int PASSES = TS / RPP;      // passes over the tile (epilogue, Cij prefetch)
  constexpr int SP = KCH / RPP;         // staging passes per chunk
  constexpr int CP = TS + VW;           // pitch of the accumulator tile in LDS
  // A staged slab row of 64 floats spans the 64 LDS banks exactly, and an 8-byte operand read is served
  // 32 lanes at a time: lanes (p, q) and (p, q+1), one slab row apart, would meet in the same banks.  Odd
  // slab rows therefore hold their two halves swapped (column ^ 32).  16-byte reads (doubles) are served
  // 16 lanes at a time, one slab row: nothing to do.
  constexpr int SWZ = sizeof(T) == 4 ? 32 : 0;
  constexpr bool TILE_IN_LAST = sizeof(T) == 8;  // which chunk requests the Cij tile, see the chunk loop
  static_assert(RPP % 2 == 0, "row parity of a staging pass");
  static_assert(KCH % RPP == 0 && KCH % 4 == 0, "chunk size");
  // LDS: the staging slabs xs | ys; once they are consumed the same memory holds the accumulator tile
  // followed by the trace reciprocals of the tile's rows and columns
  constexpr int TAIL = TS * CP + 2 * TS;
  constexpr int SLAB = 2 * KCH * TS > TAIL ? 2 * KCH * TS : TAIL;

  __shared__ __attribute__((aligned(16))) T slab[SLAB];
  T *xs = slab, *ys = slab + KCH * TS;
  T *rci_s = slab + TS * CP, *rcj_s = rci_s + TS;

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, p = lane & 15, q = lane >> 4;
  // Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.  Renumbered so that one XCD
  // gets a contiguous run of tiles.  The run walks the tile grid in panels of panel_cols tile columns,
  // row by row inside a panel, so the tiles in flight at any time share a few column slabs of y and a
  // limited set of row slabs of x.  One column per panel (column-major order) when the whole batch of x
  // fits an L2 anyway: a few hundred KB of y plus all of x per L2.  For big layers a column-major order
  // re-read x from HBM once per tile column (measured 460 GB per launch at 65536 x 100000, batch 1024).
  const unsigned ntiles = (unsigned)(a.tiles_i * a.tiles_j);  // < 2^31, checked by the launcher
  const unsigned per_xcd = (ntiles + 7) / 8;
  const unsigned tile = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (tile >= ntiles) return;  // whole workgroup, before any barrier
  const unsigned panel = a.by_panel.div(tile);
  const unsigned in_panel = tile - panel * ((unsigned)a.tiles_i * a.panel_cols);
  long it = in_panel, jt = panel;
  if (a.panel_cols > 1) {  // uniform
    const unsigned first = panel * a.panel_cols;
    const unsigned width = (unsigned)a.tiles_j - first < a.panel_cols ? (unsigned)a.tiles_j - first : a.panel_cols;
    const unsigned row = width == a.panel_cols ? in_panel >> __builtin_ctz(a.panel_cols) : in_panel / width;
    it = row;
    jt = first + (in_panel - row * width);
  }
  const long i0 = it * TS, j0 = jt * TS;

  // thread's share of the tile in row-major order: VW columns of PASSES rows
  const int eg = tid % G, er = tid / G;
  const long ecol = j0 + VW * eg;

  SB_PHASE_MARK(0);
  // x, y, the Cij tile and the W tile are reached through bounds-checked buffer windows: rows past the
  // batch or past the matrix read zero / store nothing in hardware, so there are no clamped addresses,
  // no zero-filling and no branches, and the row advance per chunk / pass is a scalar offset.  Loads
  // return in issue order, hence the order below: first what the first MFMA needs (chunk 0 of x and
  // y, mostly L2 hits), and the Cij tile (HBM) only while the second-to-last chunk is being computed.
  constexpr unsigned ES = sizeof(T);
  const long tile_rows = a.N - i0 < TS ? a.N - i0 : TS;
  const BufferWindow<T> cwin(a.Cij + i0 * a.M, tile_rows * a.M), wwin(a.W + i0 * a.M, tile_rows * a.M);
  T sx[SP][VW], sy[SP][VW];
  // byte offsets of this thread's vectors relative to the first row of a chunk
  unsigned xat[SP], yat[SP];
#pragma unroll
  for (int m = 0; m < SP; m++) {
    xat[m] = (unsigned)(((long)(er + RPP * m) * a.N + i0 + VW * eg) * ES);
    yat[m] = (unsigned)(((long)(er + RPP * m) * a.M + ecol) * ES);
  }
  auto request_chunk = [&](long b0) {
    // windows from the chunk's first batch row to the end of x / y (scalar arithmetic): rows past the
    // batch fall outside, and the per-lane offsets stay those of chunk 0 whatever the batch size
    const BufferWindow<T> xwin(a.x + b0 * a.N, (a.B - b0) * a.N), ywin(a.y + b0 * a.M, (a.B - b0) * a.M);
#pragma unroll
    for (int m = 0; m < SP; m++) {
      xwin.template load<true>(sx[m], xat[m], 0, i0 + VW * eg, a.N);
      ywin.template load<true>(sy[m], yat[m], 0, ecol, a.M);
    }
  };
  request_chunk(0);

  // column sums: one wavefront takes the 64 x columns of the tile (a lane each), one the 64 y columns,
  // the other two take none; which wavefronts do rotates with the tile, so that over the tiles of a
  // CU the work is spread over its four SIMDs
  const int role = __builtin_amdgcn_readfirstlane((w + (int)tile) & 3);
  const bool summer = role < 2;  // uniform per wavefront
  const bool sum_i = role == 0;
  const int scol = lane;
  const T *sbase = (sum_i ? xs : ys) + scol, *sbase_odd = (sum_i ? xs : ys) + (scol ^ SWZ);
  const long sidx = (sum_i ? i0 : j0) + scol;
  const bool sum_ok = summer && sidx < (sum_i ? a.N : a.M);
  const bool writes_bias = !PRE && sum_ok && !sum_i && it == 0 && a.bias_mode == 1;
  // old trace; with PRE the new one, which the same two wavefronts turn into the reciprocals below
  const T cold = (PRE ? (sum_i ? a.Ci_next : a.Cj_next) : (sum_i ? a.Ci : a.Cj))[sum_ok ? sidx : 0];
  T kb = T(1);
  if (!PRE && a.bias_mode == 1) kb = a.kbi[writes_bias ? sidx : 0];
  T csum = T(0);

  // mask bytes of the thread's PASSES x VW synapses: a small, L2-resident array, fetched up front
  uint32_t mb[PASSES][MB];
  if (a.wmask) {
    uint32_t hc[MB];
#pragma unroll
    for (int e = 0; e < MB; e++) hc[e] = ecol + e < a.M ? a.by_Mc.div((uint32_t)(ecol + e)) : 0u;
#pragma unroll
    for (int k = 0; k < PASSES; k++) {
      const long row = i0 + er + RPP * k;
#pragma unroll
      for (int e = 0; e < MB; e++) mb[k][e] = a.wmask[row < a.N ? row * a.H + hc[e] : 0];
    }
  }

  T cpre[PASSES][VW];  // Cij tile: VW columns of PASSES rows per thread
  const unsigned tat = (unsigned)(((long)er * a.M + ecol) * ES);  // this thread's vector in pass 0
  const unsigned pass_bytes = (unsigned)((long)RPP * a.M * ES);    // the next pass is RPP rows further on
  auto request_tile = [&]() {
#pragma unroll
    for (int k = 0; k < PASSES; k++) cwin.template load<true>(cpre[k], tat, k * pass_bytes, ecol, a.M);
  };

  acc_t acc[2][2];
#pragma unroll
  for (int r = 0; r < 2; r++)
#pragma unroll
    for (int c = 0; c < 2; c++) acc[r][c] = acc_t{0, 0, 0, 0};
  const int iw = (w >> 1) * 32, jw = (w & 1) * 32;  // sub-tile of this wavefront

  // ---- chunks of the batch.  The loads of chunk c+1 are issued before chunk c is consumed from LDS,
  // so their latency hides behind the MFMA loop and the column sums.
  auto chunk = [&](long b0, auto with_tile) {
    if (b0 > 0) {
      __syncthreads();  // previous chunk fully consumed
      SB_PHASE_MARK(2 * (int)(b0 / KCH));
    }
#pragma unroll
    for (int m = 0; m < SP; m++) {
      typename R::vec_t vx, vy;
#pragma unroll
      for (int e = 0; e < VW; e++) {
        vx[e] = sx[m][e];
        vy[e] = sy[m][e];
      }
      const int at = (er + RPP * m) * TS + ((VW * eg) ^ ((er & 1) * SWZ));
      *reinterpret_cast<typename R::vec_t *>(&xs[at]) = vx;
      *reinterpret_cast<typename R::vec_t *>(&ys[at]) = vy;
    }
    __syncthreads();
    SB_PHASE_MARK(1 + 2 * (int)(b0 / KCH));
    request_chunk(b0 + KCH);  // past the batch: reads zeros nobody consumes
    if (decltype(with_tile)::value) request_tile();

    if (!PRE && summer) {
      // rows past the end of the batch were staged as zeros: adding them changes nothing, so the loop
      // needs no guard; 16 LDS reads are in flight before the (ordered) additions consume them
      for (int r = 0; r < KCH; r += 16) {
        T v[16];
#pragma unroll
        for (int k = 0; k < 16; k++) v[k] = (k & 1 ? sbase_odd : sbase)[(r + k) * TS];
#pragma unroll
        for (int k = 0; k < 16; k++) csum = R::add(csum, v[k]);
      }
    }

    // K loop: per step of 4 batch rows, lane (p,q) feeds row 4s+q of the slabs.  The operands of step
    // s+1 are read from LDS before the MFMAs of step s are issued (the fences keep that order).
    const T *xa = xs + q * TS + ((iw + 2 * p) ^ ((q & 1) * SWZ));
    const T *ya = ys + q * TS + ((jw + 2 * p) ^ ((q & 1) * SWZ));
    T xo[2][2], yo[2][2];
    xo[0][0] = xa[0], xo[0][1] = xa[1], yo[0][0] = ya[0], yo[0][1] = ya[1];
#pragma unroll
    for (int s = 0; s < KCH / 4; s++) {
      const int cur = s & 1, nxt = cur ^ 1;
      if (s + 1 < KCH / 4) {
        xo[nxt][0] = xa[(s + 1) * 4 * TS], xo[nxt][1] = xa[(s + 1) * 4 * TS + 1];
        yo[nxt][0] = ya[(s + 1) * 4 * TS], yo[nxt][1] = ya[(s + 1) * 4 * TS + 1];
      }
      __builtin_amdgcn_sched_barrier(0);
      acc[0][0] = R::mfma(xo[cur][0], yo[cur][0], acc[0][0]);
      acc[0][1] = R::mfma(xo[cur][0], yo[cur][1], acc[0][1]);
      acc[1][0] = R::mfma(xo[cur][1], yo[cur][0], acc[1][0]);
      acc[1][1] = R::mfma(xo[cur][1], yo[cur][1], acc[1][1]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  long b0 = 0;
  if constexpr (TILE_IN_LAST) {
    // doubles: a chunk takes twice as long, enough to cover the tile's latency, and the tile's registers
    // then never coexist with the staging registers of a further chunk
    for (; b0 + KCH < a.B; b0 += KCH) chunk(b0, std::false_type{});
    chunk(b0, std::true_type{});
  } else {
    for (; b0 + 2 * KCH < a.B; b0 += KCH) chunk(b0, std::false_type{});
    chunk(b0, std::true_type{});  // second-to-last (or only) chunk: the Cij tile is requested here
    b0 += KCH;
    if (b0 < a.B) chunk(b0, std::false_type{});
  }

  __syncthreads();  // slabs consumed: their memory is reused from here on
  SB_PHASE_MARK(12);

  // ---- 3. new traces of this tile's rows and columns (reference order of operations)
  if (summer) {
    T cnew = T(1);
    if (sum_ok) {
      if constexpr (PRE) {
        cnew = cold;
      } else {
        cnew = trace_next<T>(cold, csum, a);
        if (sum_i) {
          if (jt == 0) a.Ci_next[sidx] = cnew;
        } else if (it == 0) {
          a.Cj_next[sidx] = cnew;
          if (writes_bias) {
            a.bias[sidx] = bias_regularized<T>(cnew, kb, a.cthr, a.khalf, a.pmin, a.taubdt);
            a.kbi[sidx] = kb;
          }
        }
      }
    }
    (sum_i ? rci_s : rcj_s)[scol] = trace_reciprocal<T>(cnew, a.cthr);
  }

  // ---- 4. accumulators -> row-major LDS tile
  T *cs = slab;
#pragma unroll
  for (int r = 0; r < 2; r++)
#pragma unroll
    for (int v = 0; v < 4; v++) {
      const int row = iw + 2 * R::acc_row(q, v) + r;
      cs[row * CP + jw + 2 * p] = acc[r][0][v];
      cs[row * CP + jw + 2 * p + 1] = acc[r][1][v];
    }
  __syncthreads();  // accumulator tile and reciprocals published
  SB_PHASE_MARK(13);

  // ---- epilogue: decay + clamp, weight, mask, stores.  Whether a synapse keeps its weight (row and
  // column above the trace threshold, mask bit set) is combined into one predicate per element.
  const T scale = a.invB * a.tau;
  const bool masked = a.wmask != nullptr;
  T rcj[VW];
  bool col_live[VW];
#pragma unroll
  for (int e = 0; e < VW; e++) {
    rcj[e] = rcj_s[VW * eg + e];
    col_live[e] = !(rcj[e] < T(0));
  }
#pragma unroll
  for (int k = 0; k < PASSES; k++) {
    const int lr = er + RPP * k;  // rows past the matrix compute garbage that the window drops
    const T rci = rci_s[lr];
    const bool row_live = !(rci < T(0)) && (MB != 1 || !masked || mb[k][0] != 0);
    T cv[VW];
#pragma unroll
    for (int e = 0; e < VW; e++) {
      const T cn = cpre[k][e] * a.omt + cs[lr * CP + VW * eg + e] * scale;
      cv[e] = fmax(cn, T(0));  // 0 as well when cn is NaN, like the reference's `cn > 0 ? cn : 0`
    }
    cwin.template store<VEC>(cv, tat, k * pass_bytes, ecol, a.M);
    // Where the mask is 0 the weight is 0, and when the caller vouches that W holds 0 there already, a
    // wavefront whose vectors all lie under zero mask bytes has nothing to compute or store.
    bool connected = !masked;
#pragma unroll
    for (int e = 0; e < MB; e++) connected = connected || mb[k][e] != 0;
    if (a.W == nullptr) continue;
    if (a.w_masked && __builtin_amdgcn_ballot_w64(connected) == 0) continue;
    T wv[VW];
#pragma unroll
    for (int e = 0; e < VW; e++) {
      const T wgt = R::wlog(fmax(cv[e], a.cthr4) * rci * rcj[e]);
      const bool keep = row_live && col_live[e] && (MB == 1 || !masked || mb[k][e] != 0);
      wv[e] = keep ? wgt : T(0);
    }
    wwin.template store<VEC>(wv, tat, k * pass_bytes, ecol, a.M);
  }
  SB_PHASE_MARK(14);
}

}  // namespace sb
