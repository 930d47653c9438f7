// Register-resident variant of the greedy swap loop of the mask rewiring (omp.cc:289-315, where
// "omp.cc" = BCPNN/backend/_kernels/kernels_openmp_internal.cc of the reference) for layers with at
// most NT*R input rows: one workgroup of NT threads, thread t owns rows t, t+NT, ...; score
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

// ---------------------------------------------------------------------------------------------------
// Fast path of the swap loop.  Over at most 16 iterations only the 16 best silent rows and the 16 worst
// active rows of the INITIAL state (plus rows that changed sides on the way) can ever be picked, because
// an iteration changes nothing but the two rows it swaps.  So:
//   phase A (whole workgroup): a radix select on monotone integer keys of the scores finds a threshold
//     per group such that the rows beyond it are a small superset of those 16; a large group of exactly
//     equal scores at the threshold (rows of dead inputs all score 0) is cut down to its highest indices,
//     which is the order the tie rule would take them in;
//   phase B (one wavefront, one candidate per lane and group): the iterations themselves, with the same
//     picks, tie rule, break conditions and score expression as the full scan.
// Anything the fast path does not cover (NaN scores, more iterations, too many near-equal candidates)
// returns false and the caller runs the full scan.
template <typename T>
struct ScoreKey;
template <>
struct ScoreKey<float> {
  using K = uint32_t;
  static constexpr int BITS = 32, PASSES = 2;
  static __device__ __forceinline__ K of(float s) {
    const uint32_t b = __float_as_uint(s + 0.0f);  // -0 and +0 compare equal, so they share a key
    return b ^ ((b >> 31) ? 0xffffffffu : 0x80000000u);
  }
};
template <>
struct ScoreKey<double> {
  using K = uint64_t;
  static constexpr int BITS = 64, PASSES = 3;
  static __device__ __forceinline__ K of(double s) {
    const uint64_t b = (uint64_t)__double_as_longlong(s + 0.0);
    return b ^ ((b >> 63) ? ~0ull : (1ull << 63));
  }
};
__device__ __forceinline__ float readlane_t(float v, int l) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l));
}
__device__ __forceinline__ double readlane_t(double v, int l) {
  const long long b = __double_as_longlong(v);
  const int lo = __builtin_amdgcn_readlane((int)(b & 0xffffffffLL), l);
  const int hi = __builtin_amdgcn_readlane((int)(b >> 32), l);
  return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}

// (key, row index) pairs and their wavefront-wide maximum; idx < 0 marks "no candidate"
template <typename K>
struct KeyIdx {
  K key;
  int idx;
};
template <typename K>
__device__ __forceinline__ KeyIdx<K> pick_key(KeyIdx<K> a, KeyIdx<K> b) {
  const bool take = b.idx >= 0 && (a.idx < 0 || b.key > a.key || (b.key == a.key && b.idx > a.idx));
  return take ? b : a;
}
__device__ __forceinline__ uint32_t readlane_k(uint32_t v, int l) {
  return (uint32_t)__builtin_amdgcn_readlane((int)v, l);
}
__device__ __forceinline__ uint64_t readlane_k(uint64_t v, int l) {
  const uint32_t lo = readlane_k((uint32_t)v, l), hi = readlane_k((uint32_t)(v >> 32), l);
  return ((uint64_t)hi << 32) | lo;
}
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_move_k(uint32_t v) {
  return (uint32_t)dpp_move<CTRL>((int)v);
}
template <int CTRL>
__device__ __forceinline__ uint64_t dpp_move_k(uint64_t v) {
  return ((uint64_t)dpp_move_k<CTRL>((uint32_t)(v >> 32)) << 32) | dpp_move_k<CTRL>((uint32_t)v);
}
template <typename K, int CTRL>
__device__ __forceinline__ KeyIdx<K> dpp_keyidx(KeyIdx<K> c) {
  return KeyIdx<K>{dpp_move_k<CTRL>(c.key), dpp_move<CTRL>(c.idx)};
}
template <typename K>
__device__ __forceinline__ KeyIdx<K> wave_pick(KeyIdx<K> c) {  // the result is wavefront-uniform
  c = pick_key<K>(c, dpp_keyidx<K, kDppSwap1>(c));
  c = pick_key<K>(c, dpp_keyidx<K, kDppSwap2>(c));
  c = pick_key<K>(c, dpp_keyidx<K, kDppHalfMirror>(c));
  c = pick_key<K>(c, dpp_keyidx<K, kDppMirror>(c));
  // every lane of a row of 16 now holds its row's pick; the four rows are combined from scalar
  // registers (a lane read is far cheaper than an exchange through the LDS crossbar)
  const KeyIdx<K> r0{readlane_k(c.key, 0), __builtin_amdgcn_readlane(c.idx, 0)};
  const KeyIdx<K> r1{readlane_k(c.key, 16), __builtin_amdgcn_readlane(c.idx, 16)};
  const KeyIdx<K> r2{readlane_k(c.key, 32), __builtin_amdgcn_readlane(c.idx, 32)};
  const KeyIdx<K> r3{readlane_k(c.key, 48), __builtin_amdgcn_readlane(c.idx, 48)};
  return pick_key<K>(pick_key<K>(r0, r1), pick_key<K>(r2, r3));
}

// 32-bit keys: (key, index + 1) packed into one 64-bit integer whose unsigned order is the order pick_key
// defines (0 = no candidate), so a pick is a 64-bit maximum: a third of the instructions.
__device__ __forceinline__ KeyIdx<uint32_t> wave_pick(KeyIdx<uint32_t> c) {
  uint64_t v = c.idx < 0 ? 0ull : ((uint64_t)c.key << 32) | (uint32_t)(c.idx + 1);
  auto larger = [](uint64_t a, uint64_t b) { return b > a ? b : a; };
  v = larger(v, dpp_move_k<kDppSwap1>(v));
  v = larger(v, dpp_move_k<kDppSwap2>(v));
  v = larger(v, dpp_move_k<kDppHalfMirror>(v));
  v = larger(v, dpp_move_k<kDppMirror>(v));
  const uint64_t m = larger(larger(readlane_k(v, 0), readlane_k(v, 16)),
                            larger(readlane_k(v, 32), readlane_k(v, 48)));
  return KeyIdx<uint32_t>{(uint32_t)(m >> 32), (int)(uint32_t)m - 1};
}

// Scatter inside a wavefront: v of every lane with `on` lands in lane `to`.  The targets must be distinct and
// must be lanes that push themselves (a permutation among the pushing lanes); the other lanes keep 0.
__device__ __forceinline__ uint32_t push_to_lane(uint32_t v, int to, bool on) {
  const int lane = (int)(threadIdx.x & 63);
  return (uint32_t)__builtin_amdgcn_ds_permute((on ? to : lane) * 4, on ? (int)v : 0);
}
__device__ __forceinline__ uint64_t push_to_lane(uint64_t v, int to, bool on) {
  return ((uint64_t)push_to_lane((uint32_t)(v >> 32), to, on) << 32) | push_to_lane((uint32_t)v, to, on);
}

__device__ __forceinline__ void note_changed(int *changed, int *nchanged, int row) {
  const int at = atomicAdd(nchanged, 1);
  if (at < kMaxChangedRows) changed[at] = row;
}

template <typename T, int NT, int R>
struct MaskSwapFast {
  using SK = ScoreKey<T>;
  using K = typename SK::K;
  static constexpr int TOPK = 16, CAP = 48, DIG = 11, BINS = 1 << DIG, PER = BINS / NT, NWV = NT / 64;
  // index bins of the tie cut: (row index) >> ISH, the smallest shift that fits NT * R rows into BINS bins
  static constexpr int ish_for(int rows) { return rows <= BINS ? 0 : 1 + ish_for((rows + 1) / 2); }
  static constexpr int ISH = ish_for(NT * R);
  static_assert(((NT * R - 1) >> ISH) < BINS && BINS % NT == 0, "row indices must fit the index histogram");
  struct Shared {
    unsigned hist[2][BINS];
    int cand[2][64], cand_cs[2][64];  // candidate rows, their connection counts ...
    T cand_nom[2][64];                // ... and score nominators
    int ncand[2], sel_bin[2], sel_above[2], wtot[2][NWV];
    K eq_min[2], eq_max[2];
  };

  // Largest bin b with (rows in bins >= b) >= need, per group; sel_bin stays -1 when the histogram holds
  // fewer than `need` rows.  Two barriers inside.
  static __device__ void crossing(Shared &sh, const int (&need)[2], const bool (&active)[2]) {
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    int c[2], incl[2];
#pragma unroll
    for (int g = 0; g < 2; g++) {
      c[g] = 0;
#pragma unroll
      for (int b = 0; b < PER; b++) c[g] += (int)sh.hist[g][PER * tid + b];
      int s = c[g];
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {  // inclusive suffix sum inside the wavefront
        const int v = __shfl_down(s, o);
        if (lane + o < 64) s += v;
      }
      incl[g] = s;
      if (lane == 0) sh.wtot[g][wv] = s;
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < 2; g++) {
      // (all totals requested at once; the ones of the wavefronts behind this one are added)
#pragma unroll
      for (int w2 = 0; w2 < NWV; w2++) {
        const int v = sh.wtot[g][w2];
        incl[g] += w2 > wv ? v : 0;
      }
      const int after = incl[g] - c[g];
      if (active[g] && after < need[g] && need[g] <= incl[g]) {  // exactly one thread per group
        int acc = after;
        for (int b = PER - 1; b >= 0; b--) {
          const int hb = (int)sh.hist[g][PER * tid + b];
          if (acc + hb >= need[g]) {
            sh.sel_bin[g] = PER * tid + b;
            sh.sel_above[g] = acc;
            break;
          }
          acc += hb;
        }
      }
    }
    __syncthreads();
  }

  static __device__ void clear(Shared &sh) {
    for (int i = threadIdx.x; i < 2 * BINS; i += NT) (&sh.hist[0][0])[i] = 0u;
    if (threadIdx.x < 2) sh.sel_bin[threadIdx.x] = -1;
  }

  // true: the swaps are done and written back; false: nothing was changed, run the full scan
  // changed / nchanged (LDS): the rows that end on the other side are appended there
  static __device__ bool run(const MaskArgs<T> &a, Shared &sh, const T (&score)[R], const int (&m)[R],
                             const T (&nom)[R], const int (&cs)[R], int *changed, int *nchanged) {
    const int tid = threadIdx.x, lane = tid & 63;
    K key[R];
#pragma unroll
    for (int k = 0; k < R; k++) {
      const K u = SK::of(score[k]);
      key[k] = m[k] == 0 ? u : (K)~u;  // in both groups the wanted rows are those with the LARGEST keys
    }
    K prefix[2] = {0, 0};
    int need[2] = {TOPK, TOPK};
    bool all[2] = {false, false};  // the whole group is wanted (it has fewer than TOPK rows)
    // ---- phase A: threshold on the leading DIG * PASSES key bits
#pragma unroll
    for (int p = 0; p < SK::PASSES; p++) {
      const int shift = SK::BITS - DIG * (p + 1);
      clear(sh);
      __syncthreads();
#pragma unroll
      for (int k = 0; k < R; k++) {
        const int g = m[k];
        if (g < 2 && !all[g] && (p == 0 || (key[k] >> (shift + DIG)) == prefix[g]))
          atomicAdd(&sh.hist[g][(unsigned)(key[k] >> shift) & (BINS - 1)], 1u);
      }
      __syncthreads();
      const bool active[2] = {!all[0], !all[1]};
      crossing(sh, need, active);
#pragma unroll
      for (int g = 0; g < 2; g++) {
        if (all[g]) continue;
        if (sh.sel_bin[g] < 0) {
          all[g] = true;
        } else {
          prefix[g] = (prefix[g] << DIG) | (K)sh.sel_bin[g];
          need[g] -= sh.sel_above[g];
        }
      }
      __syncthreads();  // everybody has read the selection before the next pass clears it
    }
    constexpr int TAIL = SK::BITS - DIG * SK::PASSES;  // key bits below the threshold's resolution
    // ---- candidates: rows at or beyond the threshold
    if (tid < 2) {
      sh.ncand[tid] = 0;
      sh.eq_min[tid] = ~(K)0;
      sh.eq_max[tid] = 0;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < R; k++) {
      const int g = m[k];
      if (g >= 2) continue;
      const K top = key[k] >> TAIL;
      if (all[g] || top >= prefix[g]) {
        const int pos = atomicAdd(&sh.ncand[g], 1);
        if (pos < 64) sh.cand[g][pos] = tid + NT * k, sh.cand_cs[g][pos] = cs[k], sh.cand_nom[g][pos] = nom[k];
      }
      if (!all[g] && top == prefix[g]) {
        atomicMin(&sh.eq_min[g], key[k]);
        atomicMax(&sh.eq_max[g], key[k]);
      }
    }
    __syncthreads();
    // ---- too many candidates: a block of exactly equal scores at the threshold is cut down to its
    // `need` highest row indices (the tie rule takes equal scores from the highest index down)
    bool cut[2];
    bool any_cut = false;
#pragma unroll
    for (int g = 0; g < 2; g++) {
      cut[g] = sh.ncand[g] > CAP;
      if (cut[g] && sh.eq_min[g] != sh.eq_max[g]) return false;  // uniform: read from LDS by everybody
      any_cut |= cut[g];
    }
    if (any_cut) {
      __syncthreads();
      clear(sh);
      if (tid < 2 && cut[tid]) sh.ncand[tid] = 0;
      __syncthreads();
#pragma unroll
      for (int k = 0; k < R; k++) {
        const int g = m[k];
        if (g < 2 && cut[g] && (key[k] >> TAIL) == prefix[g]) atomicAdd(&sh.hist[g][(tid + NT * k) >> ISH], 1u);
      }
      __syncthreads();
      crossing(sh, need, cut);
#pragma unroll
      for (int k = 0; k < R; k++) {
        const int g = m[k];
        if (g >= 2 || !cut[g]) continue;
        const K top = key[k] >> TAIL;
        const int i = tid + NT * k;
        if (top > prefix[g] || (top == prefix[g] && (i >> ISH) >= sh.sel_bin[g])) {
          const int pos = atomicAdd(&sh.ncand[g], 1);
          if (pos < 64) sh.cand[g][pos] = i, sh.cand_cs[g][pos] = cs[k], sh.cand_nom[g][pos] = nom[k];
        }
      }
      __syncthreads();
      if (sh.ncand[0] > CAP || sh.ncand[1] > CAP) return false;
    }
    if (tid >= 64) return true;  // phase B is the first wavefront's

    // ---- phase B: lane l holds silent candidate l and active candidate l.  A pick is the maximum of
    // (key, row index) pairs -- the key orders the scores, the index settles equal scores in favour of
    // the later row, as the sequential >= / <= scans do.  A row that changes sides takes the score of
    // its other side along (csum +- 1), computed once up front, so the loop holds no division.
    int nS = sh.ncand[0], nA = sh.ncand[1];
    const int nS0 = nS, nA0 = nA;  // rows that change sides are appended from these slots on
    bool vS = lane < nS, vA = lane < nA;
    int iS = vS ? sh.cand[0][lane] : 0, iA = vA ? sh.cand[1][lane] : 0;
    int csS = vS ? sh.cand_cs[0][lane] : 0, csA = vA ? sh.cand_cs[1][lane] : 0;
    const T nomS = vS ? sh.cand_nom[0][lane] : T(0), nomA = vA ? sh.cand_nom[1][lane] : T(0);
    // keys as seen from the silent side (largest score wins) and from the active side (smallest wins)
    K kS = SK::of(mask_score<T>(nomS, csS)), kS_other = (K)~SK::of(mask_score<T>(nomS, csS + 1));
    K kA = (K)~SK::of(mask_score<T>(nomA, csA)), kA_other = SK::of(mask_score<T>(nomA, csA - 1));
    // ---- All swaps at once, when that provably equals the loop below.  Rank the candidates of each side
    // by (key, row index), the order the picks take them in; iteration k of the loop then picks the
    // rank-k candidates of both sides and swaps them unless the silent one scores lower, so the number of
    // swaps n is the length of the run of such pairs from rank 0 -- provided no row that changed sides
    // is ever picked again.  That holds when every new active row scores strictly above, and every new
    // silent row strictly below, the last pair the loop would look at; otherwise (blocks of equal scores,
    // dead inputs) the loop runs.  Both sides must also hold a candidate for every iteration that happens.
    {
      const int kmax = (int)(a.iterations < (nS < nA ? nS : nA) ? a.iterations : (nS < nA ? nS : nA));
      int rS = 0, rA = 0;
      const int widest = nS > nA ? nS : nA;
      for (int m = 0; m < widest; m++) {  // uniform
        const K kSm = readlane_k(kS, m), kAm = readlane_k(kA, m);
        const int iSm = __builtin_amdgcn_readlane(iS, m), iAm = __builtin_amdgcn_readlane(iA, m);
        rS += (m < nS && (kSm > kS || (kSm == kS && iSm > iS))) ? 1 : 0;
        rA += (m < nA && (kAm > kA || (kAm == kA && iAm > iA))) ? 1 : 0;
      }
      // lane k: the score keys of the rank-k silent and rank-k active candidates
      const K sortedS = push_to_lane(kS, rS, vS), sortedA = (K)~push_to_lane(kA, rA, vA);
      const unsigned long long keep_going = __ballot(lane < kmax && !(sortedS < sortedA));
      const int n = __builtin_ctzll(~keep_going);  // (kmax <= 16: bit kmax is clear)
      const bool complete = n < kmax || kmax == (int)a.iterations;
      if (n == 0 && complete) return true;  // nothing to swap
      if (complete) {
        const int last = n < kmax ? n : kmax - 1;  // the last pair the loop looks at
        const K lastS = readlane_k(sortedS, last), lastA = readlane_k(sortedA, last);
        const bool toA = vS && rS < n, toS = vA && rA < n;
        const bool again = (toA && !((K)~kS_other > lastA)) || (toS && !(kA_other < lastS));
        if (__ballot(again) == 0) {
          if (toA) {
            a.wmask[(long)iS * a.H + a.h] = 1;
            a.csum[iS] = csS + 1;
            note_changed(changed, nchanged, iS);
          }
          if (toS) {
            a.wmask[(long)iA * a.H + a.h] = 0;
            a.csum[iA] = csA - 1;
            note_changed(changed, nchanged, iA);
          }
          return true;
        }
      }
    }
    for (long it = 0; it < a.iterations; it++) {
      KeyIdx<K> cmax{kS, vS ? iS : -1}, cmin{kA, vA ? iA : -1};
      cmax = wave_pick(cmax);
      cmin = wave_pick(cmin);
      if (cmax.idx < 0 || cmin.idx < 0) break;  // no silent or no active row
      if (cmax.key < (K)~cmin.key) break;       // vmax0 < vmin1
      const int lS = __builtin_ctzll(__ballot(vS && iS == cmax.idx));
      const int lA = __builtin_ctzll(__ballot(vA && iA == cmin.idx));
      const K wOther = readlane_k(kS_other, lS), wThis = cmax.key;  // winner: its active-side key, ...
      const K lOther = readlane_k(kA_other, lA), lThis = cmin.key;
      const int csW = __builtin_amdgcn_readlane(csS, lS), csL = __builtin_amdgcn_readlane(csA, lA);
      if (lane == lS) vS = false;
      if (lane == lA) vA = false;
      if (lane == nA) {  // the best silent row becomes active
        vA = true, iA = cmax.idx, csA = csW + 1;
        kA = wOther, kA_other = wThis;
      }
      if (lane == nS) {  // the worst active row becomes silent
        vS = true, iS = cmin.idx, csS = csL - 1;
        kS = lOther, kS_other = lThis;
      }
      nA++, nS++;
    }
    if (vS) {
      a.wmask[(long)iS * a.H + a.h] = 0;
      a.csum[iS] = csS;
      if (lane >= nS0) note_changed(changed, nchanged, iS);
    }
    if (vA) {
      a.wmask[(long)iA * a.H + a.h] = 1;
      a.csum[iA] = csA;
      if (lane >= nA0) note_changed(changed, nchanged, iA);
    }
    return true;
  }
};

// Steps 3 and 4 in the swap kernel's wake (a.W_fix != nullptr), by the whole workgroup: the weights of the
// rows that changed sides -- every other row of the hypercolumn already holds what its unchanged mask byte
// asks for -- and the hypercolumn's row list.  All threads of the workgroup call it.
template <typename T, int NT>
__device__ __forceinline__ void mask_swap_finish(const MaskArgs<T> &a, const int *changed, const int *nchanged) {
  if (a.W_fix == nullptr) return;  // uniform
  __syncthreads();                 // mask bytes and the list of changed rows are written
  if (a.rows != nullptr) mask_rows_block<NT>(a.rows, a.row_cnt, a.wmask, a.N, a.H, a.cap, a.h);
  const unsigned nc = *nchanged < kMaxChangedRows ? *nchanged : kMaxChangedRows, Mc = (unsigned)a.Mc;
  for (unsigned e = threadIdx.x; e < nc * Mc; e += NT) {
    const unsigned r = e / Mc, c = e - r * Mc;
    const long i = changed[r], j = a.h * a.Mc + c;
    T wgt = T(0);
    if (a.wmask[i * a.H + a.h] != 0)
      wgt = weight_from_traces<T>(a.Cij[i * a.M + j], trace_reciprocal<T>(a.Ci[i], a.cthr),
                                  trace_reciprocal<T>(a.Cj[j], a.cthr), a.cthr4);
    a.W_fix[i * a.M + j] = wgt;
  }
}

// NT threads (64 to 1024 in powers of two), thread t owns rows t, t+NT, ..., t+(R-1)*NT.  1024 threads
// with few rows each measured faster than 256 with more (1568 rows: 19.8 against 21.8 us).
template <typename T, int NT, int R>
__global__ __launch_bounds__(NT) void k_mask_swap_reg(MaskArgs<T> a) {
  constexpr int NWV = NT / 64;
  static_assert(NWV == 1 || NWV == 2 || NWV == 4 || NWV == 8 || NWV == 16, "1 to 16 wavefronts");
  __shared__ RowCand<T> part[2][4][NWV];  // [buffer][max0, min1, first0, first1][wavefront]
  __shared__ int changed[kMaxChangedRows], nchanged;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  if (tid == 0) nchanged = 0;  // (published by the barrier below)

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
  if (!track_first && a.iterations <= MaskSwapFast<T, NT, R>::TOPK) {
    __shared__ typename MaskSwapFast<T, NT, R>::Shared fast_lds;
    if (MaskSwapFast<T, NT, R>::run(a, fast_lds, score, m, nom, cs, changed, &nchanged)) {
      mask_swap_finish<T, NT>(a, changed, &nchanged);
      return;
    }
    __syncthreads();
  }

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
      if (NWV > 4) {  // the lanes of a quad agree by now, so mirroring 8 (16) lanes pairs the quads
        cmax = pick_max<T>(cmax, dpp_cand<kDppHalfMirror, T>(cmax));
        cmin = pick_min<T>(cmin, dpp_cand<kDppHalfMirror, T>(cmin));
        f0 = pick_first<T>(f0, dpp_cand<kDppHalfMirror, T>(f0));
        f1 = pick_first<T>(f1, dpp_cand<kDppHalfMirror, T>(f1));
      }
      if (NWV > 8) {
        cmax = pick_max<T>(cmax, dpp_cand<kDppMirror, T>(cmax));
        cmin = pick_min<T>(cmin, dpp_cand<kDppMirror, T>(cmin));
        f0 = pick_first<T>(f0, dpp_cand<kDppMirror, T>(f0));
        f1 = pick_first<T>(f1, dpp_cand<kDppMirror, T>(f1));
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
      note_changed(changed, &nchanged, (int)i);
    }
  }
  mask_swap_finish<T, NT>(a, changed, &nchanged);
}

}  // namespace sb
