// Definitions of the launchers declared in sb_launch.hpp; included once per element type by
// sb_kernels_f32.hip / sb_kernels_f64.hip, which instantiate them explicitly.
#pragma once
#include "sb_kernels.hpp"
#include "sb_k_train.hpp"
#include "sb_k_forward_rows.hpp"
#include "sb_k_skinny.hpp"
#include "sb_launch.hpp"

#include <algorithm>
#include <hip/hip_ext.h>
#include <cstdlib>

namespace sb {

static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static inline long cdiv(long a, long b) { return (a + b - 1) / b; }

#define SB_LAUNCH_CHECK() SB_HIP(hipGetLastError())

// ------------------------------------------------------------------------------------------- forward
template <typename T, int NG, bool FUSE>
static int forward_variant(hipStream_t st, ForwardArgs<T> a, bool vec) {
  ProfScope prof_(st, K_FORWARD);
  a.by_batch_tiles = FastDiv::of(a.batch_tiles);
  // 8 workgroup ids per round of XCDs; ids beyond the last tile exit at once
  const long ntiles = a.col_tiles * a.batch_tiles;
  const long grid = 8 * cdiv(ntiles, 8);
  if (grid >= (1L << 31)) {
    set_error("launch_forward: too many tiles for one launch");
    return -1;
  }
  if (vec)
    hipLaunchKernelGGL((k_forward<T, NG, FUSE, true, 8>), dim3((unsigned)grid), dim3(512), 0, st, a);
  else
    hipLaunchKernelGGL((k_forward<T, NG, FUSE, false, 8>), dim3((unsigned)grid), dim3(512), 0, st, a);
  SB_LAUNCH_CHECK();
  return 0;
}

static inline int device_cu_count() {
  static const int n = [] {
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) {
      hipDeviceProp_t prop;
      if (hipGetDeviceProperties(&prop, dev) == hipSuccess) cus = prop.multiProcessorCount;
    }
    return cus;
  }();
  return n;
}

template <typename T>
int launch_forward(hipStream_t st, T *act, const T *x, const T *W, const T *bias, long B, long N,
                   long H, long Mc, bool softmax) {
  return launch_forward_classify<T>(st, act, x, W, bias, B, N, H, Mc, softmax, nullptr, nullptr, nullptr);
}

template <typename T>
int launch_forward_classify(hipStream_t st, T *act, const T *x, const T *W, const T *bias, long B, long N,
                            long H, long Mc, bool softmax, const T *labels, int32_t *pred,
                            unsigned long long *correct) {
  constexpr int VW = Real<T>::VW;
  constexpr int GW = 16 * VW;
  SB_REQUIRE(act && x && W && bias, "null pointer");
  SB_REQUIRE(B > 0 && N > 0 && H > 0 && Mc > 0, "sizes must be positive");
  const long M = H * Mc;
  SB_REQUIRE(M < (1L << 31) && N < (1L << 31), "dimension too large");
  // A handful of output units: plain vector arithmetic, one workgroup per batch row.  Its time grows with M
  // where the MFMA kernel's is flat (3000 inputs, batch 128: float 7.1 us at M = 10, 15.6 at 32, MFMA 15.9;
  // double 12.2 at 10, 17.2 at 16, 30.9 at 32, MFMA 17.5).
  if (M <= (sizeof(T) == 4 ? 32 : 16)) {
    SB_REQUIRE(B < (1L << 31), "batch too large for one launch");
    ProfScope prof_(st, K_FORWARD);
    SB_REQUIRE(!labels || correct, "labels need a counter");
    hipLaunchKernelGGL((k_forward_skinny<T>), dim3((unsigned)B), dim3(256), 0, st, act, x, W, bias, N, M, Mc,
                       softmax ? 1 : 0, labels, pred, correct);
    SB_LAUNCH_CHECK();
    return 0;
  }
  if (labels || pred) {  // wider layers: the forward pass, then the classification kernel
    int rc = launch_forward<T>(st, act, x, W, bias, B, N, H, Mc, softmax);
    if (rc) return rc;
    return launch_argmax_rows<T>(st, act, labels, B, M, pred, correct);
  }
  // per-lane byte offsets inside one chunk of 16 rows of x or W are 32-bit
  SB_REQUIRE(16 * (N > M ? N : M) * (long)sizeof(T) < (1L << 31), "layer too wide for the forward kernel");
  ForwardArgs<T> a{act, x, W, bias, B, N, M, Mc, 0, cdiv(B, 16)};
  const bool base_vec = (N % VW == 0) && (M % VW == 0) && aligned16(x) && aligned16(W);
  const long need = cdiv(Mc, GW);
  const long max_fused = sizeof(T) == 4 ? 4 : 7;
  // The fused kernel runs one workgroup per hypercolumn and 16 batch rows, one workgroup per CU.  For wide
  // hypercolumns (more than two column groups) whose tiles fill their last round of workgroups badly,
  // tiles of two column groups plus a separate softmax pass are faster (1568 -> Hx200, batch 128, fused
  // against separate: H = 16: 31.7 / 23.4 us, H = 30: 33.9 / 40.0, H = 48: 63.4 / 57.1, H = 64: 66.1 / 74.5).
  const long fused_tiles = H * cdiv(B, 16), cus_ = device_cu_count();
  const bool enough_tiles = need <= 2 || 20 * fused_tiles >= 17 * cdiv(fused_tiles, cus_) * cus_;
  if (softmax && need <= max_fused && enough_tiles) {
    const bool vec = base_vec && (Mc % VW == 0);
    a.col_tiles = H;
    // Hypercolumns that need 7 column blocks of 16 (97..112 columns, e.g. 100): the last group runs
    // with 3 (float) or 1 (double) blocks instead of VW, provided none of its vectors straddles the
    // end of the hypercolumn.
    const long nblocks = cdiv(Mc, 16);
    if (vec && nblocks == 7) {
      constexpr int NGL = 8 / VW, LWL = 7 - (NGL - 1) * VW;  // float: 2 groups, 3 blocks; double: 4, 1
      if ((Mc - (NGL - 1) * GW) % LWL == 0) {
        // Large batches: 64 or 32 rows per workgroup instead of 16 while there still are enough tiles for
        // eight rounds / one round of workgroups, so that W crosses the L2 -> L1 path a quarter / half as
        // often (64 rows with fewer rounds lose more to the last, partly filled round than they gain).
        const long cus = device_cu_count();
        // (double: at most 32 rows, 64 do not fit the register file)
        long rb = sizeof(T) == 4 && H * cdiv(B, 64) >= 8 * cus ? 4 : (H * cdiv(B, 32) >= cus ? 2 : 1);
        // (32-bit byte offsets inside the tile's rows)
        while (rb > 1 && 16 * rb * N * (long)sizeof(T) >= (1L << 31)) rb /= 2;
        a.batch_tiles = cdiv(B, 16 * rb);
        a.by_batch_tiles = FastDiv::of(a.batch_tiles);
        ProfScope prof_(st, K_FORWARD);
        const long grid = 8 * cdiv(a.col_tiles * a.batch_tiles, 8);
        SB_REQUIRE(grid < (1L << 31), "too many tiles for one launch");
        const dim3 g((unsigned)grid);
        if constexpr (sizeof(T) == 4) {
          // 100 columns = 6 blocks of 16 + 4: the last four as 4x4 products instead of a seventh block
          if (Mc == 6 * 16 + 4) {
            if (rb == 4) hipLaunchKernelGGL((k_forward<T, 2, true, true, 8, 2, 4, true>), g, dim3(512), 0, st, a);
            else if (rb == 2) hipLaunchKernelGGL((k_forward<T, 2, true, true, 8, 2, 2, true>), g, dim3(512), 0, st, a);
            else hipLaunchKernelGGL((k_forward<T, 2, true, true, 8, 2, 1, true>), g, dim3(512), 0, st, a);
            SB_LAUNCH_CHECK();
            return 0;
          }
          if (rb == 4) hipLaunchKernelGGL((k_forward<T, NGL, true, true, 8, LWL, 4>), g, dim3(512), 0, st, a);
        }
        if (rb == 4) {
        } else if (rb == 2)
          hipLaunchKernelGGL((k_forward<T, NGL, true, true, 8, LWL, 2>), g, dim3(512), 0, st, a);
        else
          hipLaunchKernelGGL((k_forward<T, NGL, true, true, 8, LWL>), g, dim3(512), 0, st, a);
        SB_LAUNCH_CHECK();
        return 0;
      }
    }
    if (need <= 1) return forward_variant<T, 1, true>(st, a, vec);
    if (need <= 2) return forward_variant<T, 2, true>(st, a, vec);
    if (need <= 4) return forward_variant<T, 4, true>(st, a, vec);
    if constexpr (sizeof(T) == 8) return forward_variant<T, 7, true>(st, a, vec);
  }
  a.col_tiles = cdiv(M, 2 * GW);
  int rc = forward_variant<T, 2, false>(st, a, base_vec);
  if (rc) return rc;
  if (softmax) return launch_softmax<T>(st, act, B, H, Mc);
  return 0;
}

// ------------------------------------------------------------------- forward over the connected rows
template <typename T>
bool forward_rows_supported(const T *W, long N, long H, long Mc) {
  constexpr int VW = Real<T>::VW;
  const long M = H * Mc;
  return M > 32 && M % VW == 0 && Mc % VW == 0 && aligned16(W) &&
         cdiv(Mc, 16 * VW) <= (sizeof(T) == 4 ? 4 : 7) && 16 * N * (long)sizeof(T) < (1L << 31);
}

template <typename T, int NG, int LW = Real<T>::VW>
static int forward_rows_variant(hipStream_t st, ForwardRowsArgs<T> a) {
  ProfScope prof_(st, K_FORWARD);
  // four wavefronts measured best (8: 8.8 us, 4: 8.2 us, 2: 9.9 us, 16: 10.7 us at 1568 -> 30x100, density 0.1)
  constexpr int NW = 4;
  // large batches: 64 or 32 rows per workgroup while there are tiles for eight rounds / three quarters
  // of a round of workgroups (much as in launch_forward), as long as the kernel then still fits two wavefronts per SIMD:
  // two workgroups per CU with fewer rows each beat one with more (204 against 240 us at 1568 -> 30x100,
  // batch 8192; 70 against 83 us at 1568 -> 100x100 in double, batch 512)
  const long cus = device_cu_count(), H = a.f.col_tiles, B = a.f.B;
  constexpr bool fits4 = forward_rows_regs<T, NG>(4) <= kRowsRegsTwoWaves;
  long rb = fits4 && H * cdiv(B, 64) >= 8 * cus ? 4 : (4 * H * cdiv(B, 32) >= 3 * cus ? 2 : 1);
  while (rb > 1 && forward_rows_regs<T, NG>((int)rb) > kRowsRegsTwoWaves) rb /= 2;
  // (32-bit byte offsets inside the tile's rows)
  while (rb > 1 && 16 * rb * a.f.N * (long)sizeof(T) >= (1L << 31)) rb /= 2;
  a.f.batch_tiles = cdiv(B, 16 * rb);
  a.f.by_batch_tiles = FastDiv::of(a.f.batch_tiles);
  const long grid = 8 * cdiv(a.f.col_tiles * a.f.batch_tiles, 8);
  SB_REQUIRE(grid < (1L << 31), "too many tiles for one launch");
  const dim3 g((unsigned)grid), blk(64 * NW);
  if (a.xt) {  // the batch is also at hand in blocks of 16 rows
    if constexpr (fits4) {
      if (rb == 4) hipLaunchKernelGGL((k_forward_rows<T, NG, NW, 4, true, LW>), g, blk, 0, st, a);
    }
    if (rb == 4) {
    } else if (rb == 2)
      hipLaunchKernelGGL((k_forward_rows<T, NG, NW, 2, true, LW>), g, blk, 0, st, a);
    else if (a.cap <= 256)  // short lists: a segment of 256 entries (see the kernel)
      hipLaunchKernelGGL((k_forward_rows<T, NG, NW, 1, true, LW, 256>), g, blk, 0, st, a);
    else
      hipLaunchKernelGGL((k_forward_rows<T, NG, NW, 1, true, LW>), g, blk, 0, st, a);
  } else {
    if constexpr (fits4) {
      if (rb == 4) hipLaunchKernelGGL((k_forward_rows<T, NG, NW, 4, false, LW>), g, blk, 0, st, a);
    }
    if (rb == 4) {
    } else if (rb == 2)
      hipLaunchKernelGGL((k_forward_rows<T, NG, NW, 2, false, LW>), g, blk, 0, st, a);
    else if (a.cap <= 256)
      hipLaunchKernelGGL((k_forward_rows<T, NG, NW, 1, false, LW, 256>), g, blk, 0, st, a);
    else
      hipLaunchKernelGGL((k_forward_rows<T, NG, NW, 1, false, LW>), g, blk, 0, st, a);
  }
  SB_LAUNCH_CHECK();
  return 0;
}

template <typename T>
int launch_forward_rows(hipStream_t st, T *act, const T *x, const T *W, const T *bias, const int *rows,
                        const int *row_cnt, long cap, long B, long N, long H, long Mc, const T *x_blocked) {
  SB_REQUIRE(act && x && W && bias && rows && row_cnt, "null pointer");
  SB_REQUIRE(B > 0 && N > 0 && H > 0 && Mc > 0, "sizes must be positive");
  SB_REQUIRE(H * Mc < (1L << 31) && N < (1L << 31), "dimension too large");
  SB_REQUIRE(cap > 0 && cap % 16 == 0, "row lists must be padded to a multiple of 16");
  SB_REQUIRE(forward_rows_supported<T>(W, N, H, Mc), "shape not supported by the row-list forward kernel");
  ForwardRowsArgs<T> a{{act, x, W, bias, B, N, H * Mc, Mc, H, cdiv(B, 16)}, rows, row_cnt, cap, x_blocked};
  const long need = cdiv(Mc, 16 * Real<T>::VW);
  // hypercolumns of 7 column blocks of 16 (97..112 columns): the last group runs with 3 (float) or 1
  // (double) blocks, provided none of its vectors straddles the end of the hypercolumn (as in launch_forward)
  {
    constexpr int VW = Real<T>::VW, GW = 16 * VW, NGL = 8 / VW, LWL = 7 - (NGL - 1) * VW;
    if (cdiv(Mc, 16) == 7 && (Mc - (NGL - 1) * GW) % LWL == 0) return forward_rows_variant<T, NGL, LWL>(st, a);
    // and of 13 column blocks (193..208 columns, 200 among them): one block in the last group
    constexpr int NGM = 16 / VW - (VW == 2 ? 1 : 0);  // float: 4 groups (12 + 1 blocks); double: 7 (12 + 1)
    if (cdiv(Mc, 16) == 13) return forward_rows_variant<T, NGM, 1>(st, a);
  }
  if (need <= 1) return forward_rows_variant<T, 1>(st, a);
  if (need <= 2) return forward_rows_variant<T, 2>(st, a);
  if (need <= 4) return forward_rows_variant<T, 4>(st, a);
  if constexpr (sizeof(T) == 8) return forward_rows_variant<T, 7>(st, a);
  return -1;
}

template <typename T>
int launch_softmax(hipStream_t st, T *act, long B, long H, long Mc) {
  SB_REQUIRE(act, "null pointer");
  SB_REQUIRE(B > 0 && H > 0 && Mc > 0, "sizes must be positive");
  const long groups = B * H;
  SB_REQUIRE(cdiv(groups, 4) < (1L << 31), "too many groups");
  ProfScope prof_(st, K_SOFTMAX);
  hipLaunchKernelGGL((k_softmax<T>), dim3((unsigned)cdiv(groups, 4)), dim3(256), 0, st, act, groups,
                     Mc);
  SB_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------------------------- fused training
template <typename T>
int launch_train_fused(hipStream_t st, const T *x, const T *y, T *Cij, T *W, const T *Ci, const T *Cj,
                       T *Ci_next, T *Cj_next, const uint8_t *wmask, int bias_mode, T *bias, T *kbi,
                       long B, long N, long H, long Mc, T taupdt, T cthr, T khalf, T pmin, T taubdt,
                       bool w_masked, const void *prefetch, size_t prefetch_bytes) {
  constexpr int VW = Real<T>::VW;
  SB_REQUIRE(x && y && Cij && Ci && Cj && Ci_next && Cj_next, "null pointer");  // W may be null: traces only
  SB_REQUIRE(Ci != Ci_next && Cj != Cj_next, "old and new traces must be distinct buffers");
  SB_REQUIRE(bias_mode == 0 || (bias && kbi), "bias update needs bias and kbi");
  SB_REQUIRE(B > 0 && N > 0 && H > 0 && Mc > 0, "sizes must be positive");
  const long M = H * Mc;
  SB_REQUIRE(M < (1L << 31) && N < (1L << 31) && B < (1L << 31), "dimension too large");
  const TraceScalars<T> s = TraceScalars<T>::from(taupdt, cthr);
  TrainArgs<T> a;
  a.x = x; a.y = y; a.Cij = Cij; a.W = W; a.Ci = Ci; a.Cj = Cj; a.Ci_next = Ci_next; a.Cj_next = Cj_next;
  a.wmask = wmask; a.w_masked = (wmask && w_masked) ? 1 : 0;
  a.bias_mode = bias_mode; a.bias = bias; a.kbi = kbi;
  a.B = B; a.N = N; a.M = M; a.H = H; a.Mc = Mc;
  a.tau = s.tau; a.omt = s.omt; a.fB = (T)B; a.invB = (T)1 / (T)B; a.cthr = s.cthr; a.cthr4 = s.cthr4;
  // traces up to cthr^2 * 2^48 keep every argument max(Cij, cthr^4) / (Ci Cj) of the float weight
  // logarithm at or above 2^-96; doubles have no such limit
  if constexpr (sizeof(T) == 4) a.lim = s.cthr * s.cthr * 0x1p48f;
  else a.lim = (T)INFINITY;
  a.khalf = khalf; a.pmin = pmin; a.taubdt = taubdt;
  a.tiles_i = cdiv(N, 64); a.tiles_j = cdiv(M, 64);
  // tile order (see the kernel): column-major while a batch of x fits an L2 with room to spare, beyond that
  // panels of 16 tile columns while a panel's y slabs (16 x 64 columns of the batch) stay within 2 MiB, else
  // of 8.  x is fetched once per panel: at 55296 x 20000, batch 256, 7.0 GB per launch with panels of 8, 5.7 GB
  // with 16 (32: 5.8 GB); the launch takes the same time either way (4.41 / 4.43 / 4.40 ms), it is not bound by
  // that traffic.
  const bool wide_panels = 16L * 64 * B * (long)sizeof(T) <= (2L << 20);
  a.panel_cols = B * N * (long)sizeof(T) > (2L << 20) ? (wide_panels ? 16u : 8u) : 1u;
  a.by_panel = FastDiv::of(a.tiles_i * a.panel_cols); a.by_Mc = FastDiv::of(Mc);
  // (a region beyond 64 MiB would push more out of the memory-side cache than it brings in)
  const bool pf = prefetch && prefetch_bytes > 0 && prefetch_bytes <= ((size_t)64 << 20);
  a.prefetch = pf ? prefetch : nullptr;
  a.prefetch_bytes = pf ? (unsigned)prefetch_bytes : 0u;
  a.prefetch_lines = (a.prefetch_bytes + 127) / 128;
  // a line per thread: what limits a cold fetch is how many misses one CU keeps in flight (a single workgroup
  // needs 29 us for the 6272 lines of a 128 x 1568 float batch, 25 workgroups on as many CUs finish inside the
  // tiles' 15 us), so the lines are spread over as many workgroups as there are lines / 256, at most 512
  // (a multiple of 8: they come first in the grid, and the tiles behind them keep their XCDs)
  a.prefetch_groups = a.prefetch_lines ? (unsigned)std::min<long>(512, 8 * cdiv(a.prefetch_lines, 8 * 256)) : 0u;
  if (M <= 32) {  // a handful of output units: plain vector arithmetic
    const long rows = skinny_train_rows(M);
    SB_REQUIRE(cdiv(N, rows) < (1L << 31), "too many rows for one launch");
    ProfScope prof_(st, K_TRAIN_FUSED, true);
    // batch rows staged per chunk (see the kernel)
    long bc = kSkinnyLoads * (256 / rows) < kSkinnyLoads * (256 / M) ? kSkinnyLoads * (256 / rows) : kSkinnyLoads * (256 / M);
    if (bc > kSkinnyStage / (rows + M)) bc = kSkinnyStage / (rows + M);
    if (bc > ((1L << 31) - 1) / (N * (long)sizeof(T))) bc = ((1L << 31) - 1) / (N * (long)sizeof(T));
    if (bc > B) bc = B;
    SB_REQUIRE(bc >= 1, "layer too wide for the small-output training kernel");
    if (prof_.carries())
      hipExtLaunchKernelGGL((k_train_skinny<T>), dim3((unsigned)cdiv(N, rows)), dim3(256), 0, st, prof_.start(),
                            prof_.stop(), 0, a, (int)bc);
    else
      hipLaunchKernelGGL((k_train_skinny<T>), dim3((unsigned)cdiv(N, rows)), dim3(256), 0, st, a, (int)bc);
    SB_LAUNCH_CHECK();
    return 0;
  }
  SB_REQUIRE(a.tiles_i * a.tiles_j < (1L << 31) - 8, "too many tiles for one launch");
  // the kernel addresses a chunk of x and y rows and one 64-row band of Cij / W through buffer windows
  // with 32-bit offsets
  SB_REQUIRE(64 * (N > M ? N : M) * (long)sizeof(T) <= (1L << 31),
             "layer too wide: 64 rows of it must stay below 2 GiB");
  // 16-byte stores of Cij and W need rows that are whole vectors (a vector must not run into the next
  // row); loads are 16-byte accesses for every shape, and neither needs more than element alignment
  const bool vec = M % VW == 0;
  // one workgroup per tile (+ the few that prefetch, which the kernel tells apart by their index)
  const dim3 grid((unsigned)(a.tiles_i * a.tiles_j) + a.prefetch_groups);
  // batch rows per turn of two chunks.  Floats: 32, 18 KiB of LDS per workgroup, so five workgroups share a
  // CU.  Doubles: 16 -- the staging registers of two chunks of 8 rows leave the kernel without spills at four
  // wavefronts per SIMD (1 % faster than 32 at 1568 x 10000, batch 512).
  constexpr int KCH = sizeof(T) == 8 ? 16 : 32;
  const bool one_byte = Mc % VW == 0;  // every vector of VW columns lies inside one hypercolumn
  ProfScope prof_(st, K_TRAIN_FUSED, true);
  // one launch, or the sum launch and the tile launch, with the profile's events riding on them
  auto launch = [&](auto kernel, dim3 g, bool first, bool last) {
    if (prof_.carries())
      hipExtLaunchKernelGGL(kernel, g, dim3(256), 0, st, first ? prof_.start() : nullptr,
                            last ? prof_.stop() : nullptr, 0, a);
    else
      hipLaunchKernelGGL(kernel, g, dim3(256), 0, st, a);
  };
  // Every tile adds up the batch's x and y columns for its own rows and columns, which with many tile
  // rows and columns is most of the kernel's vector arithmetic (43 % at 65536 x 100000, batch 1024).
  // From one and a half rounds of workgroups on (floats; doubles: two and a half), a small launch computes the
  // new traces once and the tiles read them.  Timed, 4096 inputs, batch 128, floats, with / without that
  // launch: 23.7 / 22.5 us at 1.05 rounds, 29.3 / 29.9 at 1.5, 34.6 / 35.6 at 2, 45.5 / 48.5 at 3, 67.1 / 69.2
  // at 5; doubles: 48.1 / 47.3 at 1.6 rounds, 55.8 / 54.3 at 2, 110.3 / 113.7 at 2.5.
  const long ntiles = a.tiles_i * a.tiles_j;
  // one round: every workgroup finds a slot at once (five per CU for floats of whole vectors, else four)
  const bool one_round = ntiles <= (long)train_waves_per_simd<T, true, 1>() * device_cu_count();
  const long pre_from = sizeof(T) == 8 ? 5 * 4 : 3 * 5;  // in half workgroups per CU
  if (vec && one_byte && 2 * ntiles >= pre_from * device_cu_count()) {
    launch(k_trace_sums<T>, dim3((unsigned)(cdiv(N, 64) + cdiv(M, 64))), true, false);
    launch(k_train_fused<T, KCH, true, 1, true>, grid, false, true);
  } else if (vec && one_byte && one_round)
    launch(k_train_fused<T, KCH, true, 1, false, true>, grid, true, true);
  else if (vec && one_byte)
    launch(k_train_fused<T, KCH, true, 1>, grid, true, true);
  else if (vec)
    launch(k_train_fused<T, KCH, true, VW>, grid, true, true);
  else if (one_byte)
    launch(k_train_fused<T, KCH, false, 1>, grid, true, true);
  else
    launch(k_train_fused<T, KCH, false, VW>, grid, true, true);
  SB_LAUNCH_CHECK();
  return 0;
}

template <typename T>
int launch_weights_from_traces(hipStream_t st, T *W, const T *Ci, const T *Cj, const T *Cij, const uint8_t *wmask,
                               T cthr, long N, long H, long Mc, bool w_masked) {
  SB_REQUIRE(W && Ci && Cj && Cij, "null pointer");
  SB_REQUIRE(N > 0 && H > 0 && Mc > 0, "sizes must be positive");
  const long M = H * Mc;
  SB_REQUIRE(M < (1L << 31) && N < (1L << 31), "dimension too large");
  const TraceScalars<T> s = TraceScalars<T>::from(T(0), cthr);
  ProfScope prof_(st, K_WEIGHT_PASS);
  constexpr int VW = Real<T>::VW;
  // 16-byte vectors that lie inside one row (and one hypercolumn), and a turn's rows inside one window
  if (M % VW == 0 && (!wmask || Mc % VW == 0) && kRowsPerTurn * M * (long)sizeof(T) < (1L << 31)) {
    const long turns = cdiv(N, kRowsPerTurn);
    const dim3 grid((unsigned)cdiv(M, 256 * VW), (unsigned)(turns < 32768 ? turns : 32768));
    if (wmask)
      hipLaunchKernelGGL((k_weight_pass<T, true>), grid, dim3(256), 0, st, W, Ci, Cj, Cij, wmask, cthr, s.cthr4, N, M,
                         H, FastDiv::of(Mc), w_masked ? 1 : 0);
    else
      hipLaunchKernelGGL((k_weight_pass<T, false>), grid, dim3(256), 0, st, W, Ci, Cj, Cij, wmask, cthr, s.cthr4, N, M,
                         H, FastDiv::of(Mc), 0);
    SB_LAUNCH_CHECK();
    return 0;
  }
  hipLaunchKernelGGL((k_weights_from_traces<T>), dim3((unsigned)(N < 8192 ? N : 8192)), dim3(256), 0, st, W, Ci,
                     Cj, Cij, cthr, s.cthr4, N, M);
  SB_LAUNCH_CHECK();
  if (wmask) return launch_apply_mask<T>(st, W, wmask, N, H, Mc);
  return 0;
}

template <typename T>
int launch_add_bias(hipStream_t st, T *act, const T *bias, long B, long M) {
  SB_REQUIRE(act && bias, "null pointer");
  SB_REQUIRE(B > 0 && M > 0, "sizes must be positive");
  const long blocks = cdiv(B * M, 256) < 8192 ? cdiv(B * M, 256) : 8192;
  ProfScope prof_(st, K_UPDATE_BIAS);
  hipLaunchKernelGGL((k_add_bias<T>), dim3((unsigned)blocks), dim3(256), 0, st, act, bias, B, M);
  SB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------- bias
template <typename T>
int launch_update_bias(hipStream_t st, T *bias, const T *Cj, T cthr, long M) {
  SB_REQUIRE(bias && Cj, "null pointer");
  SB_REQUIRE(M > 0, "sizes must be positive");
  ProfScope prof_(st, K_UPDATE_BIAS);
  hipLaunchKernelGGL((k_update_bias<T>), dim3((unsigned)cdiv(M, 256)), dim3(256), 0, st, bias, Cj, cthr,
                     M);
  SB_LAUNCH_CHECK();
  return 0;
}

template <typename T>
int launch_update_bias_regularized(hipStream_t st, T *bias, T *kbi, const T *Cj, T cthr, T khalf,
                                   T pmin, T taubdt, long M) {
  SB_REQUIRE(bias && kbi && Cj, "null pointer");
  SB_REQUIRE(M > 0, "sizes must be positive");
  ProfScope prof_(st, K_UPDATE_BIAS_REG);
  hipLaunchKernelGGL((k_update_bias_regularized<T>), dim3((unsigned)cdiv(M, 256)), dim3(256), 0, st,
                     bias, kbi, Cj, cthr, khalf, pmin, taubdt, M);
  SB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------- mask
// W_fix != nullptr: the swap kernel also rewrites the weights of the rows that changed sides and (rows !=
// nullptr) rebuilds the hypercolumn's row list, when it can (*merged = true); see MaskArgs.
template <typename T>
static int update_mask_impl(hipStream_t st, uint8_t *wmask, const T *W, const T *Ci, const T *Cj,
                            const T *Cij, T cthr, long N, long H, long Mc, long h, long iterations, T *nom,
                            int *csum, T *W_fix, int *rows, int *row_cnt, long cap, bool *merged) {
  SB_REQUIRE(wmask && Ci && Cj && Cij && nom && csum, "null pointer");
  SB_REQUIRE(N > 0 && H > 0 && Mc > 0, "sizes must be positive");
  SB_REQUIRE(h >= 0 && h < H, "hypercolumn index out of range");
  SB_REQUIRE(iterations >= 0, "iterations must be non-negative");
  SB_REQUIRE(cdiv(N, 4) < (1L << 31), "in_features too large");
  const TraceScalars<T> s = TraceScalars<T>::from(T(0), cthr);
  MaskArgs<T> a;
  a.wmask = wmask; a.W = W; a.Ci = Ci; a.Cj = Cj; a.Cij = Cij; a.cthr = cthr; a.cthr4 = s.cthr4;
  a.N = N; a.M = H * Mc; a.H = H; a.Mc = Mc; a.h = h; a.iterations = iterations; a.nom = nom;
  a.csum = csum;
  // two rows change sides per iteration; the kernels for more than 65536 rows have no such tail
  const bool merge = W_fix != nullptr && iterations > 0 && 2 * iterations <= kMaxChangedRows && N <= 65536 &&
                     N * Mc < (1L << 31);
  a.W_fix = merge ? W_fix : nullptr;
  a.rows = merge ? rows : nullptr;
  a.row_cnt = row_cnt;
  a.cap = cap;
  if (merged) *merged = merge;
  {
    ProfScope prof_(st, K_MASK_SCORES);
    hipLaunchKernelGGL((k_mask_scores<T>), dim3((unsigned)cdiv(N, 4)), dim3(256), 0, st, a);
    SB_LAUNCH_CHECK();
  }
  if (iterations > 0) {
    ProfScope prof_(st, K_MASK_SWAP);
    if (N <= 2048)
      hipLaunchKernelGGL((k_mask_swap_reg<T, 1024, 2>), dim3(1), dim3(1024), 0, st, a);
    else if (N <= 8192)
      hipLaunchKernelGGL((k_mask_swap_reg<T, 1024, 8>), dim3(1), dim3(1024), 0, st, a);
    else if (N <= 32768)
      hipLaunchKernelGGL((k_mask_swap_reg<T, 1024, 32>), dim3(1), dim3(1024), 0, st, a);
    else if (N <= 65536)
      hipLaunchKernelGGL((k_mask_swap_reg<T, 1024, 64>), dim3(1), dim3(1024), 0, st, a);
    else
      hipLaunchKernelGGL((k_mask_swap<T>), dim3(1), dim3(1024), 0, st, a);
    SB_LAUNCH_CHECK();
  }
  return 0;
}

template <typename T>
int launch_update_mask(hipStream_t st, uint8_t *wmask, const T *W, const T *Ci, const T *Cj,
                       const T *Cij, T cthr, long N, long H, long Mc, long h, long iterations, T *nom,
                       int *csum) {
  return update_mask_impl<T>(st, wmask, W, Ci, Cj, Cij, cthr, N, H, Mc, h, iterations, nom, csum, nullptr,
                             nullptr, nullptr, 0, nullptr);
}

template <typename T>
int launch_rewire(hipStream_t st, uint8_t *wmask, T *W, const T *Ci, const T *Cj, const T *Cij, T cthr, long N,
                  long H, long Mc, long h, long iterations, T *nom, int *csum, int *rows, int *row_cnt,
                  long cap) {
  SB_REQUIRE(W, "null pointer");
  SB_REQUIRE(!rows || (row_cnt && cap > 0 && cap % 16 == 0), "row list arguments");
  bool merged = false;
  int rc = update_mask_impl<T>(st, wmask, (const T *)nullptr, Ci, Cj, Cij, cthr, N, H, Mc, h, iterations, nom,
                               csum, W, rows, row_cnt, cap, &merged);
  if (rc || merged) return rc;
  return launch_mask_fix_weights<T>(st, W, wmask, Ci, Cj, Cij, cthr, N, H, Mc, h, rows, row_cnt, cap);
}

template <typename T>
int launch_mask_fix_weights(hipStream_t st, T *W, const uint8_t *wmask, const T *Ci, const T *Cj,
                            const T *Cij, T cthr, long N, long H, long Mc, long h, int *rows, int *row_cnt,
                            long cap) {
  SB_REQUIRE(W && wmask && Ci && Cj && Cij, "null pointer");
  SB_REQUIRE(h >= 0 && h < H, "hypercolumn index out of range");
  SB_REQUIRE(!rows || (row_cnt && cap > 0 && cap % 16 == 0), "row list arguments");
  SB_REQUIRE(cdiv(N * Mc, 256) + 1 < (1L << 31), "too many elements for one launch");
  const TraceScalars<T> s = TraceScalars<T>::from(T(0), cthr);
  ProfScope prof_(st, K_MASK_FIX);
  // with a row list, one more workgroup rebuilds the list of hypercolumn h
  const long blocks = cdiv(N * Mc, 256) + (rows ? 1 : 0);
  hipLaunchKernelGGL((k_mask_fix_weights<T>), dim3((unsigned)blocks), dim3(256), 0, st, W, wmask, Ci, Cj, Cij,
                     cthr, s.cthr4, N, H * Mc, H, Mc, h, rows, row_cnt, cap);
  SB_LAUNCH_CHECK();
  return 0;
}

template <typename T>
int launch_apply_mask(hipStream_t st, T *W, const uint8_t *wmask, long N, long H, long Mc) {
  SB_REQUIRE(W && wmask, "null pointer");
  SB_REQUIRE(N > 0 && H > 0 && Mc > 0, "sizes must be positive");
  SB_REQUIRE(H * Mc < (1L << 31), "dimension too large");
  const long blocks = N < 8192 ? N : 8192;
  ProfScope prof_(st, K_APPLY_MASK);
  constexpr int VW = Real<T>::VW;
  if (Mc % VW == 0 && aligned16(W)) {
    const long turns = cdiv(N, kRowsPerTurn);
    hipLaunchKernelGGL((k_apply_mask_vec<T>), dim3((unsigned)cdiv(H * Mc, 256 * VW), (unsigned)(turns < 4096 ? turns : 4096)),
                       dim3(256), 0, st, W, wmask, N, H * Mc, H, FastDiv::of(Mc));
    SB_LAUNCH_CHECK();
    return 0;
  }
  hipLaunchKernelGGL((k_apply_mask<T>), dim3((unsigned)blocks), dim3(256), 0, st, W, wmask, N, H * Mc, H,
                     FastDiv::of(Mc));
  SB_LAUNCH_CHECK();
  return 0;
}

// *count += number of entries of W that are non-zero under a zero mask byte
template <typename T>
int launch_count_unmasked(hipStream_t st, const T *W, const uint8_t *wmask, long N, long H, long Mc,
                          unsigned long long *count) {
  SB_REQUIRE(W && wmask && count, "null pointer");
  SB_REQUIRE(N > 0 && H > 0 && Mc > 0, "sizes must be positive");
  SB_REQUIRE(H * Mc < (1L << 31), "dimension too large");
  const long blocks = N < 4096 ? N : 4096;
  ProfScope prof_(st, K_APPLY_MASK);
  hipLaunchKernelGGL((k_count_unmasked<T>), dim3((unsigned)blocks), dim3(256), 0, st, W, wmask, N, H * Mc, H,
                     Mc, count);
  SB_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------------------------- classification
template <typename T>
int launch_argmax_rows(hipStream_t st, const T *act, const T *labels, long B, long M, int32_t *pred,
                       unsigned long long *correct) {
  SB_REQUIRE(act, "null pointer");
  SB_REQUIRE(!labels || correct, "labels need a counter");
  SB_REQUIRE(B > 0 && M > 0, "sizes must be positive");
  ProfScope prof_(st, K_ARGMAX);
  hipLaunchKernelGGL((k_argmax_rows<T>), dim3((unsigned)cdiv(B, 4)), dim3(256), 0, st, act, labels, B,
                     M, pred, correct);
  SB_LAUNCH_CHECK();
  return 0;
}

template <typename T>
int launch_gather_rows(hipStream_t st, T *dst, const T *src, const int64_t *idx, long rows,
                       long cols) {
  SB_REQUIRE(dst && src && idx, "null pointer");
  SB_REQUIRE(rows > 0 && cols > 0 && rows < (1L << 31), "bad shape");
  ProfScope prof_(st, K_GATHER);
  hipLaunchKernelGGL((k_gather_rows<T>), dim3((unsigned)rows), dim3(256), 0, st, dst, src, idx, rows,
                     cols);
  SB_LAUNCH_CHECK();
  return 0;
}

template <typename T>
int launch_gather_rows_blocked(hipStream_t st, T *dst, T *plain, const T *src, const int64_t *idx, long rows,
                               long cols) {
  SB_REQUIRE(dst && src, "null pointer");
  SB_REQUIRE(rows > 0 && cols > 0 && cdiv(rows, 16) < (1L << 31), "bad shape");
  ProfScope prof_(st, K_GATHER);
  hipLaunchKernelGGL((k_gather_rows_blocked<T>), dim3((unsigned)cdiv(rows, 16)), dim3(256), 0, st, dst, plain,
                     src, idx, rows, cols);
  SB_LAUNCH_CHECK();
  return 0;
}

template <typename T>
int launch_mfma_probe(hipStream_t st, T *sink, long workgroups, long iters) {
  SB_REQUIRE(sink, "null pointer");
  SB_REQUIRE(workgroups > 0 && workgroups < (1L << 31) && iters > 0 && iters <= (1L << 24), "bad sizes");
  hipLaunchKernelGGL((k_mfma_probe<T>), dim3((unsigned)workgroups), dim3(256), 0, st, sink, iters);
  SB_LAUNCH_CHECK();
  return 0;
}

template <typename T>
int launch_fill(hipStream_t st, T *dst, T value, size_t n) {
  if (n == 0) return 0;
  SB_REQUIRE(dst, "null pointer");
  const size_t blocks = (n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096;
  ProfScope prof_(st, K_FILL);
  hipLaunchKernelGGL((k_fill<T>), dim3((unsigned)blocks), dim3(256), 0, st, dst, value, n);
  SB_LAUNCH_CHECK();
  return 0;
}

template <typename T>
int launch_copy_pair(hipStream_t st, T *dst1, const T *src1, size_t n1, T *dst2, const T *src2, size_t n2) {
  if (n1 + n2 == 0) return 0;
  SB_REQUIRE(dst1 && src1 && dst2 && src2, "null pointer");
  const size_t blocks = (n1 + n2 + 255) / 256 < 4096 ? (n1 + n2 + 255) / 256 : 4096;
  ProfScope prof_(st, K_FILL);
  hipLaunchKernelGGL((k_copy_pair<T>), dim3((unsigned)blocks), dim3(256), 0, st, dst1, src1, n1, dst2, src2, n2);
  SB_LAUNCH_CHECK();
  return 0;
}

#define SB_INSTANTIATE_LAUNCHERS(T)                                                                   \
  template int launch_forward<T>(hipStream_t, T *, const T *, const T *, const T *, long, long, long, \
                                 long, bool);                                                         \
  template int launch_forward_classify<T>(hipStream_t, T *, const T *, const T *, const T *, long,    \
                                          long, long, long, bool, const T *, int32_t *,               \
                                          unsigned long long *);                                      \
  template bool forward_rows_supported<T>(const T *, long, long, long);                               \
  template int launch_forward_rows<T>(hipStream_t, T *, const T *, const T *, const T *, const int *, \
                                      const int *, long, long, long, long, long, const T *);          \
  template int launch_gather_rows_blocked<T>(hipStream_t, T *, T *, const T *, const int64_t *, long, \
                                             long);                                                  \
  template int launch_softmax<T>(hipStream_t, T *, long, long, long);                                 \
  template int launch_train_fused<T>(hipStream_t, const T *, const T *, T *, T *, const T *, const T *, \
                                     T *, T *, const uint8_t *, int, T *, T *, long, long, long, long, \
                                     T, T, T, T, T, bool, const void *, size_t);                                             \
  template int launch_update_bias<T>(hipStream_t, T *, const T *, T, long);                           \
  template int launch_weights_from_traces<T>(hipStream_t, T *, const T *, const T *, const T *,       \
                                             const uint8_t *, T, long, long, long, bool);             \
  template int launch_add_bias<T>(hipStream_t, T *, const T *, long, long);                           \
  template int launch_update_bias_regularized<T>(hipStream_t, T *, T *, const T *, T, T, T, T, long); \
  template int launch_update_mask<T>(hipStream_t, uint8_t *, const T *, const T *, const T *,         \
                                     const T *, T, long, long, long, long, long, T *, int *);         \
  template int launch_mask_fix_weights<T>(hipStream_t, T *, const uint8_t *, const T *, const T *,    \
                                          const T *, T, long, long, long, long, int *, int *, long);  \
  template int launch_rewire<T>(hipStream_t, uint8_t *, T *, const T *, const T *, const T *, T, long, \
                                long, long, long, long, T *, int *, int *, int *, long);              \
  template int launch_apply_mask<T>(hipStream_t, T *, const uint8_t *, long, long, long);             \
  template int launch_count_unmasked<T>(hipStream_t, const T *, const uint8_t *, long, long, long,    \
                                        unsigned long long *);                                        \
  template int launch_argmax_rows<T>(hipStream_t, const T *, const T *, long, long, int32_t *,        \
                                     unsigned long long *);                                           \
  template int launch_gather_rows<T>(hipStream_t, T *, const T *, const int64_t *, long, long);       \
  template int launch_mfma_probe<T>(hipStream_t, T *, long, long);                                    \
  template int launch_fill<T>(hipStream_t, T *, T, size_t);                                           \
  template int launch_copy_pair<T>(hipStream_t, T *, const T *, size_t, T *, const T *, size_t);

}  // namespace sb
