// Forward pass of a structural-plasticity layer over the connected inputs only.
//
// The layer keeps W masked (apply_mask, omp.cc:322-335): W[i, columns of hypercolumn h] is zero
// wherever wmask[i, h] is 0, so in  act = softmax_per_hypercolumn(x . W + bias)  (omp.cc:70-87 +
// kernels_numpy.py:13-25) those rows add exact zeros to hypercolumn h.  With a connection density of
// 0.1 nine tenths of the reduction are such zeros.  k_forward_rows skips them: per hypercolumn it walks
// the ascending list of connected rows (k_mask_rows in sb_kernels.hpp keeps the lists in step with
// wmask) and gathers those rows of W and those columns of x.  Same tiling, accumulator layout and
// epilogue as k_forward.
#pragma once
#include "sb_k_forward.hpp"
#include "sb_kernels.hpp"

namespace sb {

template <typename T>
struct ForwardRowsArgs {
  ForwardArgs<T> f;
  const int *rows;     // [H, cap], see k_mask_rows
  const int *row_cnt;  // [H]
  long cap;            // a multiple of 16
  const T *xt;         // XT kernels: the batch in blocks of 16 rows (k_gather_rows_blocked), from row 0
};

// Wavefronts per SIMD the kernel's registers are budgeted for: three or two (as many workgroups of four
// wavefronts per CU, one computing while another waits for its gathers) where the operand ring, the
// accumulators and the x operands leave room for that, one for the big tiles.
template <typename T, int NG>
constexpr int forward_rows_regs(int rb) {  // registers of the three, in 32-bit units
  constexpr int VW = Real<T>::VW, D = sizeof(T) / 4;
  return (2 * VW * NG * VW + rb * NG * VW * 4 + 2 * rb * VW) * D;
}
constexpr int kRowsRegsTwoWaves = 150, kRowsRegsThreeWaves = 104;  // measured: no spills up to these
template <typename T, int NG, int RB>
constexpr int forward_rows_waves_per_simd() {
  constexpr int regs = forward_rows_regs<T, NG>(RB);
  return regs <= kRowsRegsThreeWaves ? 3 : regs <= kRowsRegsTwoWaves ? 2 : 1;
}

// A workgroup owns 16 batch rows x one hypercolumn (as k_forward with FUSE).  The hypercolumn's row list
// is staged through LDS in segments of SEG entries; the wavefronts split a segment in interleaved chunks
// of 4*VW entries.  Per chunk, lane (p,q) reads the VW list entries VW*q .. VW*q+VW-1 from LDS, then
// x[b0+p, row] for each of them (the A operands of VW MFMA steps) and VW*NG vectors of VW columns of
// W[row, :] (the B operands); the operands of one chunk are in flight while the previous one is
// multiplied.  A padding entry (-1) contributes x = 0 times row 0 of W (which under the kernel's
// precondition is either zero for this hypercolumn or a term of the sum anyway).  Nothing up to the first MFMAs
// depends on the hypercolumn's row count: every wavefront multiplies its first chunk of the first
// segment, which is padding where the list is shorter.
// Requires M % VW == 0, Mc % VW == 0 and 16-byte aligned W.
// RB: row blocks per workgroup, as in k_forward: 16*RB batch rows share every gathered W vector.
// XT: x is read from the blocked copy `xt` instead of a.x: the 16 lanes p of an entry then read 16
// consecutive elements (one 64-byte access) instead of one element each of 16 rows.
// LW: column blocks of the last group, as in k_forward (a hypercolumn of 100 columns takes 7 blocks of
// 16 instead of 8: the last group's lanes load LW consecutive columns).
// SEG: list entries staged per segment, 2048 or, for lists of at most 256 entries, 256: every thread loads
// and stores SEG / 256 entries per segment whatever the list's length, and at batch 128 the kernel is a
// chain of latencies that starts with this staging (1568 -> 30x100, density 0.1, lists of 157: 6.31 -> 6.13 us).
template <typename T, int NG, int NWAVES, int RB = 1, bool XT = false, int LW = Real<T>::VW, int SEG = 2048>
__global__ __launch_bounds__(64 * NWAVES)
__attribute__((amdgpu_waves_per_eu(forward_rows_waves_per_simd<T, NG, RB>(),
                                   forward_rows_waves_per_simd<T, NG, RB>())))
void k_forward_rows(ForwardRowsArgs<T> ar) {
  const ForwardArgs<T> &a = ar.f;
  constexpr int VW = Real<T>::VW;
  using TC = TileCols<T, NG, LW>;
  constexpr int KC = 4 * VW;      // list entries per chunk
  constexpr int SEGC = SEG / KC;  // chunks per segment
  static_assert(SEGC >= NWAVES && SEG % (64 * NWAVES) == 0, "segment size");
  using acc_t = typename Real<T>::acc_t;
  using vec_t = typename Real<T>::vec_t;
  typedef int ivec_t __attribute__((ext_vector_type(VW)));
  // (the short-list variant is the one whose time is a chain of latencies: its partial sums meet in LDS in one
  // step instead of two, 6.14 -> 6.06 us at 1568 -> 30x100, batch 128)
  constexpr int NT = SEG == 256 ? NWAVES : NWAVES / 2;
  __shared__ __attribute__((aligned(16))) T red[NT][16][TC::CP];
  __shared__ __attribute__((aligned(16))) int sidx[SEG];

  // XCD-aware renumbering, as in k_forward
  const long ntiles = a.col_tiles * a.batch_tiles;
  const long per_xcd = (ntiles + 7) / 8;
  const long tile = (long)(blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (tile >= ntiles) return;  // whole workgroup, before any barrier
  const long ct = a.by_batch_tiles.div((uint32_t)tile), bt = tile - ct * a.batch_tiles;  // tile < 2^31

  const int tid = threadIdx.x, lane = tid & 63, p = lane & 15, q = lane >> 4;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const long b0 = bt * (16 * RB);
  const long j0 = ct * a.Mc;
  const long ncol = a.Mc;
  const int *list = ar.rows + ct * ar.cap;

  // first segment of the list on its way before anything else
  constexpr int PT = SEG / (64 * NWAVES);  // entries per thread and segment
  int mine[PT];
  auto request_segment = [&](long seg0) {
#pragma unroll
    for (int t = 0; t < PT; t++) {
      const long k = seg0 + tid + t * (64 * NWAVES);
      mine[t] = list[k < ar.cap ? k : 0];  // entries past the list are replaced by padding below
    }
  };
  auto publish_segment = [&](long seg0) {
#pragma unroll
    for (int t = 0; t < PT; t++) {
      const long k = seg0 + tid + t * (64 * NWAVES);
      sidx[tid + t * (64 * NWAVES)] = k < ar.cap ? mine[t] : -1;
    }
  };
  request_segment(0);
  const int cnt = ar.row_cnt[ct];

  acc_t acc[RB][NG][VW];
#pragma unroll
  for (int r = 0; r < RB; r++)
#pragma unroll
    for (int g = 0; g < NG; g++)
#pragma unroll
      for (int c = 0; c < VW; c++) acc[r][g][c] = acc_t{0, 0, 0, 0};

  T bv[ForwardBias<T, NG, NWAVES>::PT];
  ForwardBias<T, NG, NWAVES>::load(bv, a.bias, j0, ncol);

  // x through a bounds-checked window over this tile's batch rows: rows past the batch and padding
  // entries (offset kOutside) read zero.  Blocked copy: block b0/16 + r starts N*16 elements after the
  // previous one, lane p's row is element p of a column's run of 16.
  const BufferWindow<T> xwin((XT ? ar.xt : a.x) + b0 * a.N,
                             (XT ? (a.B + 15) / 16 * 16 - b0 : a.B - b0) * a.N);
  unsigned xat[RB];
#pragma unroll
  for (int r = 0; r < RB; r++)
    xat[r] = XT ? (unsigned)(((long)r * a.N * 16 + p) * sizeof(T))
                : (unsigned)((long)(16 * r + p) * a.N * sizeof(T));
  constexpr unsigned XSTEP = (XT ? 16u : 1u) * (unsigned)sizeof(T);  // bytes between input columns
  // W: this lane's columns of group g, or the tile's first columns where the group hangs over the end
  // of the hypercolumn (those accumulator columns are never stored)
  const T *wcol[NG];
#pragma unroll
  for (int g = 0; g < NG; g++) wcol[g] = a.W + j0 + (TC::gcol(g, p) < ncol ? TC::gcol(g, p) : 0);

  T xr[2][RB][VW];
  T wr[2][VW][NG][VW];
  // operands of chunk c of the staged segment (c past the segment: its last chunk again, never used)
  auto request = [&](int c, T(&xo)[RB][VW], T(&wo)[VW][NG][VW]) {
    const ivec_t idx = *reinterpret_cast<const ivec_t *>(&sidx[(c < SEGC ? c : SEGC - 1) * KC + VW * q]);
#pragma unroll
    for (int s = 0; s < VW; s++) {
      const int r = idx[s];
#pragma unroll
      for (int rb = 0; rb < RB; rb++) {
        T one[1];
        xwin.template load_n<1>(one, r < 0 ? BufferWindow<T>::kOutside : xat[rb] + (unsigned)r * XSTEP);
        xo[rb][s] = one[0];
      }
      const long roff = (long)(r < 0 ? 0 : r) * a.M;
#pragma unroll
      for (int g = 0; g < NG; g++) {
        if (TC::gwidth(g) == VW) {
          const vec_t v = *reinterpret_cast<const vec_t *>(wcol[g] + roff);
#pragma unroll
          for (int c2 = 0; c2 < VW; c2++) wo[s][g][c2] = v[c2];
        } else {
          const PackedCols<T, LW> v = *reinterpret_cast<const PackedCols<T, LW> *>(wcol[g] + roff);
#pragma unroll
          for (int c2 = 0; c2 < LW; c2++) wo[s][g][c2] = v.v[c2];
        }
      }
    }
  };
  auto compute = [&](const T(&xi)[RB][VW], const T(&wi)[VW][NG][VW]) {
#pragma unroll
    for (int s = 0; s < VW; s++)
#pragma unroll
      for (int g = 0; g < NG; g++)
#pragma unroll
        for (int c = 0; c < VW; c++)
          if (c < TC::gwidth(g)) {
#pragma unroll
            for (int r = 0; r < RB; r++) acc[r][g][c] = Real<T>::mfma(xi[r][s], wi[s][g][c], acc[r][g][c]);
          }
  };

  for (long seg0 = 0;;) {
    publish_segment(seg0);
    __syncthreads();
    request(w, xr[0], wr[0]);  // this wavefront's first chunk of the segment
    // chunks w, w + NWAVES, ... of the segment that hold list entries: n of them (at least 1 in the
    // first segment, see above)
    const long left = (long)cnt - seg0;  // entries from the start of this segment
    const long segc = left >= SEG ? SEGC : (left + KC - 1) / KC;
    long n = w < segc ? (segc - 1 - w) / NWAVES + 1 : 0;
    if (seg0 == 0 && n == 0) n = 1;
    const bool more = left > SEG;
    if (more) request_segment(seg0 + SEG);  // uniform
    __builtin_amdgcn_sched_barrier(0);
    long i = 0;
    for (; i + 2 <= n; i += 2) {
      // the scheduling fences keep the requests where they are written, ahead of the MFMAs
      request(w + (int)(i + 1) * NWAVES, xr[1], wr[1]);
      __builtin_amdgcn_sched_barrier(0);
      compute(xr[0], wr[0]);
      __builtin_amdgcn_sched_barrier(0);
      request(w + (int)(i + 2) * NWAVES, xr[0], wr[0]);
      __builtin_amdgcn_sched_barrier(0);
      compute(xr[1], wr[1]);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (i < n) compute(xr[0], wr[0]);
    if (!more) break;
    seg0 += SEG;
    __syncthreads();  // everyone is done with the staged segment
  }
#pragma unroll
  for (int r = 0; r < RB; r++) {
    if (r > 0) __syncthreads();  // the previous row block's sums have been read
    forward_finish<T, NG, true, NWAVES, LW, false, NT>(acc[r], bv, red, a.act, a.B, a.M, b0 + 16 * r, j0, ncol);
  }
}

}  // namespace sb
