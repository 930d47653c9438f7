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
// A workgroup (256 threads, 4 wavefronts) owns a 64 x 64 tile of Cij; 18 KiB of LDS and at most 96
// registers per thread let five workgroups share a CU, so the 1175 tiles of a 1568 x 3000 layer are
// all resident at once.
//   1. Per chunk of KCH / 2 batch rows it stages x[:, i-tile] and y[:, j-tile] in LDS.  x and y are
//      "k-major" in memory, which is the 16x16x4 MFMA operand layout, so staging is a plain copy.  Each
//      wavefront owns 16 rows x 64 columns of the tile (4 MFMA blocks) and feeds them with one element
//      of x and one 16-byte vector of y per lane and K step of 4; the block columns are interleaved so
//      that a lane's results of a row are consecutive columns, and the tile is loaded, updated and
//      stored as 16-byte vectors straight from the accumulator registers (no pass through LDS).  The
//      slabs are double-buffered and the global loads of two chunks are in flight: chunk c is staged from
//      its registers, the registers take the loads of chunk c+2, and one barrier per chunk separates the
//      staging from the MFMA loop (at the start, chunk 1 is requested only once chunk 0 has been staged).
//   2. From the same LDS slabs, the lanes of one wavefront add up one column each of x, those of
//      another one column each of y (which two wavefronts rotates with the tile index), in batch order
//      b = 0..B-1 without FMA contraction: the reference's summation order, so Ci, Cj and kbi stay
//      bit-exact against a strict-IEEE build of it.  Every tile needs Ci for its rows and Cj
//      for its columns, so every workgroup recomputes them from the OLD traces (a tile row shares x,
//      a tile column shares y: same inputs, same order, same bits).  The old traces are read from
//      Ci/Cj and the new ones written to Ci_next/Cj_next by the tiles of the first tile column / row:
//      no workgroup ever reads a value another one is writing.
//   3. Global loads return in issue order, so the Cij tile (HBM latency) is requested only with two or
//      three chunks left, behind the loads of the last chunk: the MFMA loop never waits for it, and it has
//      arrived by the time the epilogue needs it.  All loads are branch-free (bounds-checked buffer windows
//      instead of guards): a guarded load makes the compiler wait for every outstanding load at the
//      join.
//   4. Epilogue per 16-byte vector: decay + clamp, weight, mask, one store each to Cij and W.  The
//      kernel is bound by instruction issue (matrix and vector instructions share the SIMD's issue
//      slots), so the common case -- no trace of the tile's rows and columns below the threshold, no
//      logarithm argument near the denormal range, which the two summing wavefronts establish for the
//      whole tile -- runs a short form of the weight expression (5 vector instructions per synapse), and
//      with w_masked a wavefront whose vectors all lie under zero mask bytes skips the weight altogether.
#pragma once
#include <type_traits>

#include "sb_kernels.hpp"

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
  T lim;  // traces up to lim (and from cthr) allow the short form of the weight expression, see the kernel
  T khalf, pmin, taubdt;
  long tiles_i, tiles_j;
  FastDiv by_panel, by_Mc;  // divisions by tiles_i * panel_cols and by Mc
  unsigned panel_cols;      // tile order: panels of this many tile columns (a power of two), see the kernel
  // Memory the next launches will read first (the next batch of inputs), or nullptr: a few extra workgroups
  // touch one element of each of its 128-byte lines, which brings them from HBM into the memory-side cache
  // (the L2s keep nothing across launches).
  const void *prefetch;
  unsigned prefetch_bytes;  // at most 64 MiB
  unsigned prefetch_lines, prefetch_groups;  // 128-byte lines of the region; workgroups that touch them
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

// The new traces Ci_next, Cj_next (and the regularized bias) on their own: what every tile of k_train_fused
// otherwise repeats for its own 64 rows and 64 columns.  Launched ahead of k_train_fused<.., PRE = true> when a
// layer has so many tiles that the repetition costs more than a launch.  A workgroup takes 64 columns of x or
// of y.  The sums keep the reference's order (batch row by batch row, one rounded addition each), which is a
// chain of B dependent additions per column; what the kernel can do is keep the memory latency out of that
// chain: all 256 threads load the next 64 batch rows (16 independent loads each) into registers while 64 of
// them add up the previous 64 rows from LDS, where the block was put down ahead of a barrier.  (1568 x 10000
// doubles, batch 512: 27 -> 12 us, which is the 47 MB of x and y at 4 TB/s; a second block in flight: slower.)
constexpr int kSumRows = 64;  // batch rows per block
template <typename T>
__global__ __launch_bounds__(256) void k_trace_sums(TrainArgs<T> a) {
  using R = Real<T>;
  __shared__ T block[2][kSumRows][64];
  const int tid = threadIdx.x, col = tid & 63, sub = tid >> 6;  // thread (sub, col) loads rows sub, sub + 4, ..
  const long groups_i = (a.N + 63) / 64;
  const bool is_i = (long)blockIdx.x < groups_i;
  const long width = is_i ? a.N : a.M;
  const long idx = (is_i ? (long)blockIdx.x : (long)blockIdx.x - groups_i) * 64 + col;
  const T *const src = is_i ? a.x : a.y;
  constexpr int PER = kSumRows / 4;  // loads per thread and block
  const unsigned es = sizeof(T);
  T v[PER];
  auto request = [&](long b0) {
    // a window over the block's rows (below 2 GiB: the launcher checks 64 rows of the wider matrix); rows
    // past the batch lie outside it and read zero, like the columns past the matrix
    const long rows = a.B - b0 < kSumRows ? a.B - b0 : kSumRows;
    const BufferWindow<T> win(uniform_pointer(src + b0 * width),
                              typename BufferWindow<T>::Bytes{(unsigned)(rows * width * es)});
#pragma unroll
    for (int k = 0; k < PER; k++) {
      const long r = sub + 4 * k;
      T one[1];
      win.template load_n<1>(one, idx < width ? (unsigned)((r * width + idx) * es) : BufferWindow<T>::kOutside);
      v[k] = one[0];
    }
  };
  request(0);
  T sum = T(0);
  int buf = 0;
  for (long b0 = 0; b0 < a.B; b0 += kSumRows, buf ^= 1) {
#pragma unroll
    for (int k = 0; k < PER; k++) block[buf][sub + 4 * k][col] = v[k];
    if (b0 + kSumRows < a.B) request(b0 + kSumRows);  // (uniform) in flight during the additions below
    __syncthreads();  // the block is there; the buffer written next time round was read before this barrier
    if (sub == 0) {
      constexpr int U = 8;
      for (int r = 0; r < kSumRows; r += U) {
        T w[U];
#pragma unroll
        for (int k = 0; k < U; k++) w[k] = block[buf][r + k][col];
#pragma unroll
        for (int k = 0; k < U; k++) sum = R::add(sum, w[k]);  // (zeros past the batch change nothing)
      }
    }
  }
  if (sub != 0 || idx >= width) return;
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
// per CU; left alone the compiler takes more registers than that allows).  Floats: five for the variant that
// layers of whole vectors take (it fits 96 registers without spilling; left alone the compiler takes 100 and
// loses the fifth workgroup), four for the others (which would spill at five).
template <typename T, bool VEC, int MB>
constexpr int train_waves_per_simd() { return sizeof(T) == 8 ? 4 : (VEC && MB == 1 ? 5 : 4); }

// VEC: Cij and W are stored as 16-byte vectors (M a multiple of VW), element by element otherwise.  Loads
// are 16-byte accesses either way: one that runs over the end of a row of x, y or Cij fetches elements of
// the next row into tile rows / columns outside the matrix, which are never stored or summed.
// MB: mask bytes fetched per vector of VW columns -- 1 when Mc is a multiple of VW (every vector lies
// inside one hypercolumn), VW otherwise.
// PRE: Ci_next and Cj_next already hold the new traces (k_trace_sums): no column sums here.
// LATE1: the second chunk of the batch is requested only once the first has been staged (see the kernel).
template <typename T, int KCH, bool VEC, int MB, bool PRE = false, bool LATE1 = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(train_waves_per_simd<T, VEC, MB>())))
void k_train_fused(TrainArgs<T> a) {
  using R = Real<T>;
  using acc_t = typename R::acc_t;
  using vec_t = typename R::vec_t;
  constexpr int VW = R::VW;             // elements per 16-byte vector
  constexpr int TS = 64;                // tile side
  constexpr int G = TS / VW;            // 16-byte groups per slab row
  constexpr int RPP = 256 / G;          // slab rows the workgroup stages per pass
  constexpr int KC = KCH / 2;           // batch rows per chunk (two chunks' loads in flight, two slab buffers)
  constexpr int SP = KC / RPP;          // staging passes per chunk
  constexpr int NG = 4 / VW;            // 16-byte vectors of a tile row held by one lane
  // The x slab has a pitch of 80 elements: lane (p, q) of wavefront w reads element 16 w + p of slab row
  // 4 s + q, and with a pitch of 64 the four q of a column would meet in one LDS bank.
  constexpr int XP = TS + 16;
  constexpr int SUMB = 8;               // LDS reads of the column sums in flight at a time
  constexpr unsigned ES = sizeof(T);
  constexpr unsigned kOutside = BufferWindow<T>::kOutside;
  static_assert(KC % RPP == 0 && KC % 4 == 0, "chunk size");

  __shared__ __attribute__((aligned(16))) T xs2[2][KC * XP];
  __shared__ __attribute__((aligned(16))) T ys2[2][KC * TS];
  __shared__ __attribute__((aligned(16))) T rci_s[TS];
  __shared__ __attribute__((aligned(16))) T rcj_s[TS];
  __shared__ int slow_s[2];

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, p = lane & 15, q = lane >> 4;
  // Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.  Renumbered so that one XCD
  // gets a contiguous run of tiles.  The run walks the tile grid in panels of panel_cols tile columns,
  // row by row inside a panel, so the tiles in flight at any time share a few column slabs of y and a
  // limited set of row slabs of x.  One column per panel (column-major order) when the whole batch of x
  // fits an L2 anyway: a few hundred KB of y plus all of x per L2.  For big layers a column-major order
  // re-read x from HBM once per tile column (measured 460 GB per launch at 65536 x 100000, batch 1024).
  // The grid has one workgroup per tile; XCD x = blockIdx % 8 holds tiles_of(x) = ntiles / 8 (+1 for
  // x < ntiles % 8) consecutive tiles.
  const unsigned ntiles = (unsigned)a.tiles_i * (unsigned)a.tiles_j;  // < 2^31, checked by the launcher
  // The first workgroups of the grid (the launcher adds them when there is something to prefetch; a multiple
  // of 8, so that the tiles keep their XCDs) touch one element
  // of every 128-byte line of the region, a lane per line, and leave: the lines come from HBM into the
  // memory-side cache while the tiles compute.  A cold line takes microseconds to arrive, which is why no
  // tile does this on the side -- its own loads, which return in issue order, would queue behind.
  if (blockIdx.x < a.prefetch_groups) {  // uniform
    const __amdgpu_buffer_rsrc_t pwin = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(a.prefetch), 0,
                                                                          (int)a.prefetch_bytes, 0x00020000);
    const unsigned first = blockIdx.x * 256 + tid;
    uint32_t sum = 0;
    for (unsigned line = first; line < a.prefetch_lines; line += a.prefetch_groups * 256)
      sum += __builtin_amdgcn_raw_buffer_load_b32(pwin, (int)(line * 128u), 0, 0);
    asm volatile("" ::"v"(sum));  // (the loads have a consumer)
    return;
  }
  const unsigned wg = blockIdx.x - a.prefetch_groups;
  const unsigned xcd = wg & 7, rem = ntiles & 7;
  const unsigned tile = xcd * (ntiles >> 3) + (xcd < rem ? xcd : rem) + (wg >> 3);
  unsigned it, jt;
  if (a.panel_cols == 1) {  // uniform
    jt = a.by_panel.div(tile);
    it = tile - jt * (unsigned)a.tiles_i;
  } else {
    const unsigned panel = a.by_panel.div(tile);
    const unsigned in_panel = tile - panel * ((unsigned)a.tiles_i * a.panel_cols);
    const unsigned first = panel * a.panel_cols;
    const unsigned width = (unsigned)a.tiles_j - first < a.panel_cols ? (unsigned)a.tiles_j - first : a.panel_cols;
    it = width == a.panel_cols ? in_panel >> __builtin_ctz(a.panel_cols) : in_panel / width;
    jt = first + (in_panel - it * width);
  }
  // every index below fits 32 bits: N, M < 2^31 and 64 rows of x, y, Cij or W stay below 2 GiB (launcher)
  const unsigned N = (unsigned)a.N, M = (unsigned)a.M;
  const unsigned i0 = it * TS, j0 = jt * TS;

  // ---- staging: thread (er, eg) copies vector eg of slab rows er, er + RPP, .. of x and of y per chunk.
  // x, y, the Cij tile and the W tile are reached through bounds-checked buffer windows: rows past the
  // batch or past the matrix read zero / store nothing in hardware, so there are no clamped addresses,
  // no zero-filling and no branches; a vector whose first column lies outside the matrix gets an offset
  // beyond every window.  Loads return in issue order, hence the order below: first what the first MFMA
  // needs (chunk 0 of x and y, mostly L2 hits), and the Cij tile (HBM) only late in the chunk loop.
  const unsigned eg = tid % G, er = tid / G;
  const unsigned xat = i0 + VW * eg < N ? (er * N + i0 + VW * eg) * ES : kOutside;
  const unsigned yat = j0 + VW * eg < M ? (er * M + j0 + VW * eg) * ES : kOutside;
  const unsigned xstep = RPP * N * ES, ystep = RPP * M * ES;  // the next staging pass (uniform)
  T sx[2][SP][VW], sy[2][SP][VW];  // two register sets: the loads of two chunks are in flight
  // Windows over the rows of one chunk: rows past the batch fall outside, and the per-lane offsets stay
  // those of chunk 0 whatever the batch size.  The chunk's first row advances by pointer; sizes are
  // 32-bit (KCH rows of x or y stay below 2 GiB).
  const T *xnext = a.x, *ynext = a.y;
  unsigned rows_left = (unsigned)a.B;  // B < 2^31 (launcher)
  auto request_chunk = [&](auto set) {
    constexpr int S = decltype(set)::value;
    const unsigned rows = rows_left < (unsigned)KC ? rows_left : (unsigned)KC;
    const BufferWindow<T> xwin(xnext, typename BufferWindow<T>::Bytes{rows * N * ES}),
        ywin(ynext, typename BufferWindow<T>::Bytes{rows * M * ES});
#pragma unroll
    for (int m = 0; m < SP; m++) {
      xwin.load_vec(sx[S][m], xat, m * xstep);
      ywin.load_vec(sy[S][m], yat, m * ystep);
    }
    xnext += KC * N;
    ynext += KC * M;
    rows_left -= rows;
  };
  // LATE1 (launches whose workgroups all fit the CUs at once): only chunk 0 is requested here; chunk 1 follows
  // once chunk 0 sits in LDS (see `chunk`).  The workgroups of a CU then start together, and what they wait for
  // first is chunk 0: with both chunks requested up front the CU's first-slab traffic doubles and the first
  // MFMAs start later (1568 x 3000, batch 128: 0.25 us per launch; the mask bytes and old traces, which only
  // the epilogue needs, likewise wait until the tile is requested: another 0.1 us).  With several rounds of
  // workgroups a new workgroup starts beside others in full swing, and the earlier request is the better one
  // (55296 x 20000, batch 256: 4.39 against 4.45 ms).
  request_chunk(std::integral_constant<int, 0>{});
  if constexpr (!LATE1) request_chunk(std::integral_constant<int, 1>{});

  // ---- this lane's share of the tile, in the layout the MFMA leaves it in: wavefront w owns tile rows
  // 16 w .. 16 w + 15 and all 64 columns as four 16 x 16 blocks; the B operand of block c is column
  // 16 VW (c / VW) + VW p + c % VW, so a lane's VW results of a row are VW consecutive columns: the tile
  // is loaded, updated and stored as 16-byte vectors straight from the accumulators.  acc[c][v] is row
  // acc_row(q, v), i.e. rows r0 + rstep v of the wavefront's 16.
  constexpr int rstep = sizeof(T) == 4 ? 1 : 4;
  const unsigned r0 = 16 * w + (sizeof(T) == 4 ? 4 * q : q);
  const long tile_rows = (long)N - i0 < TS ? (long)N - i0 : TS;
  const unsigned tile_bytes = (unsigned)tile_rows * M * ES;  // at most 2 GiB (launcher)
  const BufferWindow<T> cwin(a.Cij + (long)i0 * a.M, typename BufferWindow<T>::Bytes{tile_bytes}),
      wwin(a.W + (long)i0 * a.M, typename BufferWindow<T>::Bytes{a.W ? tile_bytes : 0u});
  unsigned tat[NG], ecol[NG];  // byte offset of row r0 of the lane's vectors inside the windows
#pragma unroll
  for (int g = 0; g < NG; g++) {
    ecol[g] = j0 + 16 * VW * g + VW * p;
    tat[g] = ecol[g] < M ? (r0 * M + ecol[g]) * ES : kOutside;
  }
  const unsigned vstep = rstep * M * ES;  // from acc[..][v] to acc[..][v + 1] (uniform)

  // mask bytes of the lane's synapses: a small, L2-resident array, requested up front, or (LATE1) together
  // with the Cij tile
  const bool masked = a.wmask != nullptr;
  uint32_t mb[4][NG][MB];
  auto request_mask = [&]() {
    const ByteWindow mwin(masked ? a.wmask + (long)i0 * a.H : nullptr, tile_rows * a.H);
    const unsigned H = (unsigned)a.H;
#pragma unroll
    for (int g = 0; g < NG; g++)
#pragma unroll
      for (int e = 0; e < MB; e++) {
        const unsigned hc = ecol[g] + e < M ? a.by_Mc.div(ecol[g] + e) : 0u;
#pragma unroll
        // (the row step goes into the per-lane offset, which the window's range check covers; the instruction's
        // scalar offset is added after that check)
        for (int v = 0; v < 4; v++) mb[v][g][e] = mwin.load((r0 + v * rstep) * H + hc, 0);
      }
  };

  // column sums: one wavefront takes the 64 x columns of the tile (a lane each), one the 64 y columns,
  // the other two take none; which wavefronts do rotates with the tile, so that over the tiles of a
  // CU the work is spread over its four SIMDs
  const int role = __builtin_amdgcn_readfirstlane((w + (int)tile) & 3);
  const bool summer = role < 2;  // uniform per wavefront
  const bool sum_i = role == 0;
  const unsigned sidx = (sum_i ? i0 : j0) + lane;
  const bool sum_ok = summer && sidx < (sum_i ? N : M);
  const bool writes_bias = !PRE && sum_ok && !sum_i && it == 0 && a.bias_mode == 1;
  // old trace; with PRE the new one, which the same two wavefronts turn into the reciprocals below
  // (requested where the mask bytes are; unguarded, like every load here)
  T cold = T(0), kb = T(1);
  auto request_old_traces = [&]() {
    cold = (PRE ? (sum_i ? a.Ci_next : a.Cj_next) : (sum_i ? a.Ci : a.Cj))[sum_ok ? sidx : 0];
    if (!PRE && a.bias_mode == 1) kb = a.kbi[writes_bias ? sidx : 0];
  };
  T csum = T(0);

  T cpre[4][NG][VW];  // Cij tile
  if constexpr (!LATE1) {
    request_mask();
    request_old_traces();
  }
  auto request_tile = [&]() {
    if constexpr (LATE1) {
      request_mask();
      request_old_traces();
    }
#pragma unroll
    for (int v = 0; v < 4; v++)
#pragma unroll
      for (int g = 0; g < NG; g++) {
        // A window of its own per row step, starting v row steps into the tile and shorter by as much: an
        // instruction's scalar offset is added after the range check, so with the step passed there a lane whose
        // first row is the tile's last would read rows past the tile (past the matrix, in the last tile row).
        const unsigned skip = v * vstep;
        const unsigned left = __builtin_amdgcn_readfirstlane(tile_bytes > skip ? tile_bytes - skip : 0u);
        const BufferWindow<T> win(uniform_pointer(a.Cij + (long)i0 * a.M + (long)v * rstep * a.M),
                                  typename BufferWindow<T>::Bytes{left});
        win.load_vec(cpre[v][g], tat[g], 0);
      }
  };

  acc_t acc[4];
#pragma unroll
  for (int c = 0; c < 4; c++) acc[c] = acc_t{0, 0, 0, 0};

  // ---- new traces of this tile's rows and columns (reference order of operations), their reciprocals
  // for the weights, and whether the tile can take the short form of the weight expression: every row
  // and column trace at or above the threshold (no weight forced to zero) and small enough that no
  // argument of the logarithm can fall below 2^-96 (max(Cij, cthr^4) / (Ci Cj) >= cthr^4 / lim^2).
  auto finish_traces = [&]() {
    T cnew = T(1);
    bool odd = false;
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
      odd = !(cnew >= a.cthr) || !(cnew <= a.lim);
    }
    (sum_i ? rci_s : rcj_s)[lane] = trace_reciprocal<T>(cnew, a.cthr);
    if (lane == 0) slow_s[role] = 0;
    if (odd) slow_s[role] = 1;
  };

  // ---- chunks of the batch, KC rows each.  Chunk c is staged from register set c % 2 into slab buffer c % 2;
  // the registers then take the loads of chunk c + 2, so two chunks are always on their way and a chunk's
  // loads have two chunks' worth of MFMAs to arrive in.  One barrier per chunk: it publishes the slab, and
  // since every wavefront reaches it only after its MFMA loop over the previous chunk, the buffer written in
  // the next turn (read last two chunks ago) is free by then.
  long t = 1;  // turn of two chunks
  auto chunk = [&](auto set, auto with_tile, auto last, auto first) {
    constexpr int S = decltype(set)::value;
    T *xs = xs2[S], *ys = ys2[S];
#pragma unroll
    for (int m = 0; m < SP; m++) {
      vec_t vx, vy;
#pragma unroll
      for (int e = 0; e < VW; e++) {
        vx[e] = sx[S][m][e];
        vy[e] = sy[S][m][e];
      }
      *reinterpret_cast<vec_t *>(&xs[(er + RPP * m) * XP + VW * eg]) = vx;
      *reinterpret_cast<vec_t *>(&ys[(er + RPP * m) * TS + VW * eg]) = vy;
    }
    // The batch's first chunk is the one that requests chunk 1 (`first`: 0 never the first chunk, 1 always, 2
    // in the first turn of the loop over turns).  The request has to stay behind the staging stores above:
    // moved up by the compiler, ahead of the wait for chunk 0, it would be the early request again -- the
    // uniform branch and the scheduling fence keep it in place.
    if constexpr (LATE1 && decltype(first)::value == 2) {
      if (t == 1) request_chunk(std::integral_constant<int, 1>{});
    } else if constexpr (LATE1 && decltype(first)::value == 1) {
      __builtin_amdgcn_sched_barrier(0);
      request_chunk(std::integral_constant<int, 1>{});
    }
    request_chunk(set);  // chunk c + 2; past the batch: reads zeros nobody consumes
    if (decltype(with_tile)::value) request_tile();
    __syncthreads();

    if (!PRE && summer) {
      // Every addition below depends on the one before it.  Beside wavefronts that stream MFMAs such a chain
      // advances by one addition per MFMA slot at best (a vector instruction that is not ready the moment
      // the previous one retires queues behind the next MFMA on the SIMD's issue port), and at the default
      // priority it also queues behind the other wavefronts' vector work, while the rest of the workgroup
      // waits at the next barrier.  So in single precision the summing wavefronts run at the highest
      // priority here, and above the others through their MFMA loop, in which they start late (in double
      // precision, where an MFMA slot is three times as long, the same change costs 1 %, so the priorities
      // stay as they are there).
      if constexpr (sizeof(T) == 4) __builtin_amdgcn_s_setprio(3);
      // rows past the end of the batch were staged as zeros: adding them changes nothing, so the loops
      // need no guard; the LDS reads are in flight before the (ordered) additions consume them
      // (two copies so that the slab pitch is a constant and the reads take immediate offsets)
      if (sum_i) {
        for (int r = 0; r < KC; r += SUMB) {
          T v[SUMB];
#pragma unroll
          for (int k = 0; k < SUMB; k++) v[k] = xs[(r + k) * XP + lane];
#pragma unroll
          for (int k = 0; k < SUMB; k++) csum = R::add(csum, v[k]);
        }
      } else {
        for (int r = 0; r < KC; r += SUMB) {
          T v[SUMB];
#pragma unroll
          for (int k = 0; k < SUMB; k++) v[k] = ys[(r + k) * TS + lane];
#pragma unroll
          for (int k = 0; k < SUMB; k++) csum = R::add(csum, v[k]);
        }
      }
    }

    // after the last chunk's sums the new traces are complete: the two summing wavefronts turn them into
    // reciprocals for the weights while the others are still multiplying
    if (decltype(last)::value && summer) finish_traces();
    if constexpr (sizeof(T) == 4 && !PRE) {
      if (summer) __builtin_amdgcn_s_setprio(1);
    }

    // K loop: per step of 4 batch rows, lane (p, q) feeds slab row 4 s + q: one element of x, NG vectors
    // of y.  The operands of step s+1 are read from LDS before the MFMAs of step s are issued (the
    // fences keep that order).
    const T *xa = xs + q * XP + 16 * w + p;
    const T *ya = ys + q * TS + VW * p;
    T xo[2];
    vec_t yo[2][NG];
    xo[0] = xa[0];
#pragma unroll
    for (int g = 0; g < NG; g++) yo[0][g] = *reinterpret_cast<const vec_t *>(ya + 16 * VW * g);
#pragma unroll
    for (int s = 0; s < KC / 4; s++) {
      const int cur = s & 1, nxt = cur ^ 1;
      if (s + 1 < KC / 4) {
        xo[nxt] = xa[(s + 1) * 4 * XP];
#pragma unroll
        for (int g = 0; g < NG; g++)
          yo[nxt][g] = *reinterpret_cast<const vec_t *>(ya + (s + 1) * 4 * TS + 16 * VW * g);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int c = 0; c < 4; c++) acc[c] = R::mfma(xo[cur], yo[cur][c / VW][c % VW], acc[c]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // Two chunks per turn, so that register sets and slab buffers have fixed names; a batch that is not a
  // whole number of turns ends in a chunk of zeros.  The Cij tile (HBM latency) is requested late -- in
  // single precision with three chunks left, in double precision, where a chunk takes twice as long and the
  // tile's registers should not coexist with the staging registers of further chunks, with two -- and right
  // after the loads of a chunk: loads return in issue order, so no chunk waits for the tile.  The turns from
  // the request on are written out, so that every load sits in straight-line code (at a join the compiler
  // would wait for all outstanding loads).
  constexpr std::integral_constant<int, 0> set0{};
  constexpr std::integral_constant<int, 1> set1{};
  constexpr std::false_type no{};
  constexpr std::true_type yes{};
  const long turns = (a.B + 2 * KC - 1) / (2 * KC);
  constexpr std::integral_constant<int, 0> f0{};
  constexpr std::integral_constant<int, 1> f1{};
  constexpr std::integral_constant<int, 2> f2{};
  if constexpr (!LATE1) {
    if constexpr (sizeof(T) == 8) {
      for (; t < turns; t++) {
        chunk(set0, no, no, f0);
        chunk(set1, no, no, f0);
      }
      chunk(set0, yes, no, f0);
      chunk(set1, no, yes, f0);
    } else {
      for (; t + 1 < turns; t++) {
        chunk(set0, no, no, f0);
        chunk(set1, no, no, f0);
      }
      if (turns >= 2) {
        chunk(set0, no, no, f0);
        chunk(set1, yes, no, f0);
        chunk(set0, no, no, f0);
        chunk(set1, no, yes, f0);
      } else {
        chunk(set0, yes, no, f0);
        chunk(set1, no, yes, f0);
      }
    }
  } else
  if constexpr (sizeof(T) == 8) {
    if (turns >= 2) {
      for (; t < turns; t++) {
        chunk(set0, no, no, f2);
        chunk(set1, no, no, f0);
      }
      chunk(set0, yes, no, f0);
      chunk(set1, no, yes, f0);
    } else {
      chunk(set0, yes, no, f1);
      chunk(set1, no, yes, f0);
    }
  } else {
    if (turns >= 3) {
      for (; t + 1 < turns; t++) {
        chunk(set0, no, no, f2);
        chunk(set1, no, no, f0);
      }
      chunk(set0, no, no, f0);
      chunk(set1, yes, no, f0);
      chunk(set0, no, no, f0);
      chunk(set1, no, yes, f0);
    } else if (turns == 2) {
      chunk(set0, no, no, f1);
      chunk(set1, yes, no, f0);
      chunk(set0, no, no, f0);
      chunk(set1, no, yes, f0);
    } else {
      chunk(set0, yes, no, f1);
      chunk(set1, no, yes, f0);
    }
  }

  // ---- epilogue: decay + clamp and the Cij stores first (they need nothing from the other wavefronts),
  // then, once the reciprocals are published, weight, mask and the W stores
  const T scale = a.invB * a.tau;
  T cn[4][NG][VW];
#pragma unroll
  for (int v = 0; v < 4; v++)
#pragma unroll
    for (int g = 0; g < NG; g++) {
      T cv[VW];
#pragma unroll
      for (int e = 0; e < VW; e++) {
        cn[v][g][e] = cpre[v][g][e] * a.omt + acc[g * VW + e][v] * scale;
        cv[e] = fmax(cn[v][g][e], T(0));  // 0 as well when cn is NaN, like the reference's `cn > 0 ? cn : 0`
      }
      if (VEC) cwin.store_vec(cv, tat[g], v * vstep);
      else cwin.template store<false>(cv, tat[g], v * vstep, ecol[g], a.M);
    }
  if (a.W == nullptr) return;  // (uniform) traces only

  __syncthreads();  // reciprocals and flags published
  T rci[4];
  vec_t rcj[NG];
#pragma unroll
  for (int v = 0; v < 4; v++) rci[v] = rci_s[r0 + rstep * v];
#pragma unroll
  for (int g = 0; g < NG; g++) rcj[g] = *reinterpret_cast<const vec_t *>(&rcj_s[16 * VW * g + VW * p]);
  const bool slow = __builtin_amdgcn_readfirstlane(slow_s[0] | slow_s[1]) != 0;

  if (VEC && MB == 1 && !slow) {
    // short form: no row or column is dead, no argument is tiny; a vector lies in one hypercolumn.
    // Where the mask is 0 the weight is 0, and when the caller vouches that W holds 0 there already,
    // such vectors are not stored, and a wavefront without a connected vector computes nothing.
#pragma unroll
    for (int v = 0; v < 4; v++)
#pragma unroll
      for (int g = 0; g < NG; g++) {
        const bool connected = !masked || mb[v][g][0] != 0;
        if (a.w_masked && __builtin_amdgcn_ballot_w64(connected) == 0) continue;
        T wv[VW];
#pragma unroll
        // (max(max(cn, 0), cthr^4) = max(cn, cthr^4), cthr^4 as well when cn is NaN)
        for (int e = 0; e < VW; e++)
          wv[e] = R::wlog_normal(R::max_floor(cn[v][g][e], a.cthr4) * rci[v] * rcj[g][e]);
        if (!a.w_masked) {  // uniform
#pragma unroll
          for (int e = 0; e < VW; e++) wv[e] = connected ? wv[e] : T(0);
        }
        wwin.store_vec(wv, (a.w_masked && !connected) ? kOutside : tat[g], v * vstep);
      }
    return;
  }

  // general form: whether a synapse keeps its weight (row and column above the trace threshold, mask
  // bit set) is combined into one predicate per element
#pragma unroll
  for (int v = 0; v < 4; v++)
#pragma unroll
    for (int g = 0; g < NG; g++) {
      const bool row_live = !(rci[v] < T(0)) && (MB != 1 || !masked || mb[v][g][0] != 0);
      bool connected = !masked;
#pragma unroll
      for (int e = 0; e < MB; e++) connected = connected || mb[v][g][e] != 0;
      if (a.w_masked && __builtin_amdgcn_ballot_w64(connected) == 0) continue;
      T wv[VW];
#pragma unroll
      for (int e = 0; e < VW; e++) {
        const T wgt = R::wlog(R::max_floor(cn[v][g][e], a.cthr4) * rci[v] * rcj[g][e]);
        const bool keep = row_live && !(rcj[g][e] < T(0)) && (MB == 1 || !masked || mb[v][g][e] != 0);
        wv[e] = keep ? wgt : T(0);
      }
      wwin.template store<VEC>(wv, tat[g], v * vstep, ecol[g], a.M);
    }
}

}  // namespace sb
