// Shared device-side types for the gfx950 BCPNN kernels: per-dtype MFMA traits and small helpers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sb {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef double f64x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// Real<T>: everything the kernels need to know about one element type.
//   VW       elements per 16-byte vector (global loads/stores move VW elements per lane)
//   mfma     D = A(16x4) * B(4x16) + C on one wavefront; lane l feeds A[l%16][l/16] and B[l/16][l%16]
//   acc_row  row of the 16x16 result held in accumulator register v of a lane in lane-group q=l/16
//            (measured on gfx950: f32 -> 4*q+v, f64 -> 4*v+q); the column is always l%16
template <typename T>
struct Real;

template <>
struct Real<float> {
  static constexpr int VW = 4;
  using vec_t = f32x4;
  using acc_t = f32x4;
  static __device__ __forceinline__ acc_t mfma(float a, float b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
  }
  // Sixteen independent 4x4x1 products on one wavefront: block l/4 gets D[i][j] += A[i] * B[j] with A[i] from
  // lane 4 (l/4) + i, B[j] from lane 4 (l/4) + j; D[i][j] is element i of lane 4 (l/4) + j's result.  With
  // the operand registers of the 16x16x4 form (lane (p, q): row p, reduction index q) the blocks are
  // (q, p / 4): rows 4 (p/4) .. +3 times 4 columns, one reduction index each; the four q are added afterwards.
  static __device__ __forceinline__ acc_t mfma_4x4(float a, float b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_4x4x1f32(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ int acc_row(int q, int v) { return 4 * q + v; }
  static __device__ __forceinline__ float log_(float x) { return logf(x); }
  // log for the weight recompute: the hardware log2 (1 ulp, v_log_f32) scaled by ln 2.  That
  // instruction flushes arguments below the normal range, so small arguments are scaled by 2^32 first
  // and 32 ln 2 is taken off again.
  static __device__ __forceinline__ float wlog(float x) {
    const bool tiny = x < 0x1p-96f;
    const float l2 = __builtin_amdgcn_logf(x * (tiny ? 0x1p32f : 1.0f));
    return __builtin_fmaf(l2, 0.693147180559945309f, tiny ? -32.0f * 0.693147180559945309f : 0.0f);
  }
  // max(x, floor) for floor >= 0, floor as well when x is NaN; one instruction (the median of x, floor and
  // +inf; fmax would first quiet a signalling NaN with an instruction of its own)
  static __device__ __forceinline__ float max_floor(float x, float floor) {
    return __builtin_amdgcn_fmed3f(x, floor, __builtin_inff());
  }
  // the same for arguments known to be at least 2^-96 (bit-identical to wlog there)
  static __device__ __forceinline__ float wlog_normal(float x) {
#pragma clang fp contract(off)
    return __builtin_amdgcn_logf(x) * 0.693147180559945309f;
  }
  static __device__ __forceinline__ float exp_(float x) { return expf(x); }
  // exp for the softmax of the fused forward kernels, arguments <= 0: the hardware exp2 on x log2(e).  The
  // product is rounded once, so the result is off by up to |x| 2^-24 relative -- below 1e-7 absolute for
  // every x <= 0, which is what a softmax output is judged by.
  static __device__ __forceinline__ float exp_nonpos(float x) {
    return __builtin_amdgcn_exp2f(x * 1.44269504088896341f);
  }
  // single IEEE operations: the pragma keeps the compiler from contracting them into FMAs
  static __device__ __forceinline__ float add(float a, float b) {
#pragma clang fp contract(off)
    return a + b;
  }
  static __device__ __forceinline__ float mul(float a, float b) {
#pragma clang fp contract(off)
    return a * b;
  }
  static __device__ __forceinline__ float div(float a, float b) {
#pragma clang fp contract(off)
    return a / b;
  }
};

template <>
struct Real<double> {
  static constexpr int VW = 2;
  using vec_t = f64x2;
  using acc_t = f64x4;
  static __device__ __forceinline__ acc_t mfma(double a, double b, acc_t c) {
    return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ int acc_row(int q, int v) { return 4 * v + q; }
  static __device__ __forceinline__ double log_(double x) { return log(x); }
  // log for the weight recompute, for positive normal finite x: the classic argument reduction
  // x = 2^k (1 + f), sqrt(1/2) <= 1 + f < sqrt(2), s = f / (2 + f), log(1 + f) = f - f^2/2 + s (f^2/2 + R(s^2)) with
  // the degree-7 minimax polynomial R of Sun's freely distributable libm (error below 2^-58), the quotient from
  // the hardware reciprocal with one Newton step and one correction of s.  Within 0.75 ulp of the exact logarithm
  // (40 million arguments against an 80-bit reference) at about a third of the library routine's instructions,
  // which is what the training kernel's epilogue spends most of its vector time on at doubles.
  static __device__ __forceinline__ double wlog_normal(double x) {
    int k = __builtin_amdgcn_frexp_exp(x);
    double m = __builtin_amdgcn_frexp_mant(x);  // in [0.5, 1)
    const bool low = m < 0.70710678118654752440;
    m = low ? m + m : m;
    k = low ? k - 1 : k;
    const double f = m - 1.0, d = 2.0 + f;
    double r = __builtin_amdgcn_rcp(d);
    r = __builtin_fma(__builtin_fma(-d, r, 1.0), r, r);
    double q = f * r;
    q = __builtin_fma(__builtin_fma(-d, q, f), r, q);
    const double z = q * q, w = z * z;
    const double t1 = w * __builtin_fma(w, __builtin_fma(w, 1.531383769920937332e-01, 2.222219843214978396e-01),
                                        3.999999999940941908e-01);
    const double t2 = z * __builtin_fma(w, __builtin_fma(w, __builtin_fma(w, 1.479819860511658591e-01,
                                                                         1.818357216161805012e-01),
                                                         2.857142874366239149e-01), 6.666666666666735130e-01);
    const double R = t2 + t1, hfsq = 0.5 * f * f, dk = (double)k;
    // k ln 2 in two parts, the high one with zeros in its last bits so that k times it is exact
    return __builtin_fma(dk, 6.93147180369123816490e-01,
                         -((hfsq - __builtin_fma(q, hfsq + R, dk * 1.90821492927058770002e-10)) - f));
  }
  // the same for any argument (bit-identical to wlog_normal where that applies); zero, subnormal, infinite, negative
  // and NaN arguments go to the library routine
  static __device__ __forceinline__ double wlog(double x) {
    return (x >= 0x1p-1022 && x < __builtin_inf()) ? wlog_normal(x) : log(x);
  }
  static __device__ __forceinline__ double max_floor(double x, double floor) { return fmax(x, floor); }
  static __device__ __forceinline__ double exp_(double x) { return exp(x); }
  static __device__ __forceinline__ double exp_nonpos(double x) { return exp(x); }
  static __device__ __forceinline__ double add(double a, double b) {
#pragma clang fp contract(off)
    return a + b;
  }
  static __device__ __forceinline__ double mul(double a, double b) {
#pragma clang fp contract(off)
    return a * b;
  }
  static __device__ __forceinline__ double div(double a, double b) {
#pragma clang fp contract(off)
    return a / b;
  }
};

// Loads VW consecutive elements row[col .. col+VW) into out[]; elements at or beyond `limit`, or the
// whole vector when !row_ok, read as zero.  VEC promises 16-byte alignment of row+col and
// limit % VW == 0, so a vector is entirely inside or entirely outside.
template <typename T, bool VEC>
__device__ __forceinline__ void load_vw(T (&out)[Real<T>::VW], const T *row, long col, long limit,
                                        bool row_ok) {
  constexpr int VW = Real<T>::VW;
  if (VEC) {
    typename Real<T>::vec_t v = {};
    if (row_ok && col < limit) v = *reinterpret_cast<const typename Real<T>::vec_t *>(row + col);
#pragma unroll
    for (int e = 0; e < VW; e++) out[e] = v[e];
  } else {
#pragma unroll
    for (int e = 0; e < VW; e++) out[e] = (row_ok && col + e < limit) ? row[col + e] : T(0);
  }
}

// A pointer whose value is the same in every lane, moved to scalar registers (the compiler does not always
// see that it is, and a buffer descriptor built from vector registers costs a loop over the distinct values).
template <typename T>
__device__ __forceinline__ T *uniform_pointer(T *p) {
  const unsigned long long b = reinterpret_cast<unsigned long long>(p);
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)b);
  const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(b >> 32));
  return reinterpret_cast<T *>(((unsigned long long)hi << 32) | lo);
}

// A bounds-checked window of at most 2 GiB onto a global array, addressed through a buffer descriptor
// with 32-bit byte offsets: a per-lane offset plus a wavefront-uniform one that lives in a scalar
// register.  Accesses past the end of the window read zero and store nothing, in hardware; so a loop
// over rows needs neither clamped addresses nor zero-filling nor branches, and advancing to the next
// rows costs no vector instruction.  A lane whose vector lies outside the array in a way the window's
// end does not express (a column beyond the row length) passes kOutside as its offset.
template <typename T>
struct BufferWindow {
  static constexpr unsigned kOutside = 0x80000000u;  // beyond any window, also after adding a uniform offset
  __amdgpu_buffer_rsrc_t rsrc;
  __device__ BufferWindow(const T *base, long elems) {
    // window size = clamp(elems * sizeof(T), 0, 2 GiB)
    const long bytes = elems > 0 ? elems * (long)sizeof(T) : 0;
    const unsigned size = (unsigned)(bytes < 0x80000000L ? bytes : 0x80000000L);
    // descriptor word 3 = 0x00020000: raw buffer, 32-bit data format, as for every untyped gfx9 buffer
    rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(base), 0, (int)size, 0x00020000);
  }
  // the same for a caller that has the size in bytes at hand (at most 2 GiB)
  struct Bytes { unsigned n; };
  __device__ BufferWindow(const T *base, Bytes bytes) {
    rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(base), 0, (int)bytes.n, 0x00020000);
  }
  using u4 = unsigned __attribute__((ext_vector_type(4)));
  using u2 = unsigned __attribute__((ext_vector_type(2)));
  // `at`: byte offset of the vector's first element (ignored parts: see `col`, `limit`); VEC moves the
  // VW elements as one 16-byte access (all or none by `col`), otherwise element by element with elements
  // at columns >= limit excluded.  A 16-byte access needs element alignment only, and the window's range
  // check applies to each of its dwords on its own: the part inside the window is read or written, the
  // rest reads zero / is dropped (measured on gfx950).
  template <bool VEC>
  __device__ __forceinline__ void load(T (&out)[Real<T>::VW], unsigned at, unsigned uniform, long col,
                                       long limit) const {
    constexpr int VW = Real<T>::VW;
    if (VEC) {
      const u4 raw = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)(col < limit ? at : kOutside),
                                                           (int)uniform, 0);
      const typename Real<T>::vec_t v = __builtin_bit_cast(typename Real<T>::vec_t, raw);
#pragma unroll
      for (int e = 0; e < VW; e++) out[e] = v[e];
    } else {
#pragma unroll
      for (int e = 0; e < VW; e++) {
        const int o = (int)(col + e < limit ? at + e * (unsigned)sizeof(T) : kOutside);
        if constexpr (sizeof(T) == 4)
          out[e] = __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b32(rsrc, o, (int)uniform, 0));
        else
          out[e] = __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b64(rsrc, o, (int)uniform, 0));
      }
    }
  }
  // one unconditional 16-byte access at byte offset `at` + `uniform` (kOutside as `at`: no access)
  __device__ __forceinline__ void load_vec(T (&out)[Real<T>::VW], unsigned at, unsigned uniform) const {
    const u4 raw = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)at, (int)uniform, 0);
    const typename Real<T>::vec_t v = __builtin_bit_cast(typename Real<T>::vec_t, raw);
#pragma unroll
    for (int e = 0; e < Real<T>::VW; e++) out[e] = v[e];
  }
  // Cache policy of the 16-byte stores: sc1 (agent scope), which writes through the XCD's L2 as the store
  // happens.  With the default policy the tens of megabytes a training launch writes stay dirty in L2 until
  // the end of the kernel, where writing them back is serial time (1568 x 3000 layer, batch 128: 18.9 us per
  // launch with the default policy, 17.1 with sc1; non-temporal: 18.7; sc1 + non-temporal: 22.5).
  static constexpr int kStoreAux = 16;
  // Stores add the uniform offset to the per-lane one and leave the instruction's scalar offset at zero:
  // the hardware fetches the data registers of a 16-byte store a few cycles after issue, and the compiler
  // keeps the following instructions from overwriting them only for stores without a scalar offset
  // register (with one, the first vector instruction after the store clobbered the data of its last lanes
  // whenever the memory pipeline was busy -- seen on gfx950 as wrong elements 1 and 2 of stored vectors).
  __device__ __forceinline__ void store_vec(const T (&in)[Real<T>::VW], unsigned at, unsigned uniform) const {
    typename Real<T>::vec_t v;
#pragma unroll
    for (int e = 0; e < Real<T>::VW; e++) v[e] = in[e];
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u4, v), rsrc, (int)(at + uniform), 0, kStoreAux);
  }
  // NE consecutive elements (4, 8, 12 or 16 bytes) as one access; element-aligned
  template <int NE>
  __device__ __forceinline__ void load_n(T (&out)[NE], unsigned at) const {
    constexpr int BYTES = NE * (int)sizeof(T);
    static_assert(BYTES == 4 || BYTES == 8 || BYTES == 12 || BYTES == 16, "one buffer access");
    using u3 = unsigned __attribute__((ext_vector_type(3)));
    unsigned raw[BYTES / 4];
    if constexpr (BYTES == 4) {
      raw[0] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)at, 0, 0);
    } else if constexpr (BYTES == 8) {
      const u2 v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, (int)at, 0, 0);
      raw[0] = v[0], raw[1] = v[1];
    } else if constexpr (BYTES == 12) {
      const u3 v = __builtin_amdgcn_raw_buffer_load_b96(rsrc, (int)at, 0, 0);
      raw[0] = v[0], raw[1] = v[1], raw[2] = v[2];
    } else {
      const u4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)at, 0, 0);
      raw[0] = v[0], raw[1] = v[1], raw[2] = v[2], raw[3] = v[3];
    }
    __builtin_memcpy(out, raw, BYTES);
  }
  template <bool VEC>
  __device__ __forceinline__ void store(const T (&in)[Real<T>::VW], unsigned at, unsigned uniform, long col,
                                        long limit) const {
    constexpr int VW = Real<T>::VW;
    if (VEC) {
      typename Real<T>::vec_t v;
#pragma unroll
      for (int e = 0; e < VW; e++) v[e] = in[e];
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u4, v), rsrc,
                                             (int)((col < limit ? at : kOutside) + uniform), 0, kStoreAux);
    } else if (col + VW <= limit) {
      // (rows that are no whole number of vectors: only the last vector of a row runs over its end, so
      // in all but the last tile column this branch is taken by every lane)
      typename Real<T>::vec_t v;
#pragma unroll
      for (int e = 0; e < VW; e++) v[e] = in[e];
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u4, v), rsrc, (int)(at + uniform), 0, kStoreAux);
    } else {
#pragma unroll
      for (int e = 0; e < VW; e++) {
        const int o = (int)(col + e < limit ? at + e * (unsigned)sizeof(T) : kOutside);
        if constexpr (sizeof(T) == 4)
          __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, in[e]), rsrc, o, (int)uniform, kStoreAux);
        else
          __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u2, in[e]), rsrc, o, (int)uniform, kStoreAux);
      }
    }
  }
};

// A raw byte window (for mask bytes): bounds-checked like BufferWindow.
struct ByteWindow {
  __amdgpu_buffer_rsrc_t rsrc;
  __device__ ByteWindow(const uint8_t *base, long bytes) {
    const long b = (base && bytes > 0) ? bytes : 0;
    rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(base), 0,
                                             (int)(unsigned)(b < 0x80000000L ? b : 0x80000000L), 0x00020000);
  }
  __device__ __forceinline__ uint32_t load(unsigned at, unsigned uniform) const {
    return __builtin_amdgcn_raw_buffer_load_b8(rsrc, (int)at, (int)uniform, 0);
  }
};

// Exchange inside a row of 16 lanes with data-parallel-primitive moves (no LDS round trip).  The four
// controls below -- swap neighbours, swap pairs, mirror each half row, mirror the row -- applied in
// turn with a commutative pick leave the row-wide result in every one of the 16 lanes.
constexpr int kDppSwap1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppSwap2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // row_half_mirror
constexpr int kDppMirror = 0x140;      // row_mirror
template <int CTRL>
__device__ __forceinline__ int dpp_move(int v) {
  return __builtin_amdgcn_update_dpp(v, v, CTRL, 0xF, 0xF, false);
}
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(dpp_move<CTRL>(__float_as_int(v)));
}
template <int CTRL>
__device__ __forceinline__ double dpp_move(double v) {
  const long long b = __double_as_longlong(v);
  const int lo = dpp_move<CTRL>((int)(b & 0xffffffffLL)), hi = dpp_move<CTRL>((int)(b >> 32));
  return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}
// op-reduction over each row of 16 lanes; every lane of the row ends with the result
template <typename T, typename Op>
__device__ __forceinline__ T row16_reduce(T v, Op op) {
  v = op(v, dpp_move<kDppSwap1>(v));
  v = op(v, dpp_move<kDppSwap2>(v));
  v = op(v, dpp_move<kDppHalfMirror>(v));
  v = op(v, dpp_move<kDppMirror>(v));
  return v;
}

// Division of n < 2^31 by a divisor fixed per launch, as a multiplication: the host prepares
// m = ceil(2^k / d) with k = 31 + ceil(log2 d), and  n / d == (n * m) >> k  for every n < 2^31
// (m * d - 2^k < 2^(k-31)).  Three instructions instead of the two dozen of a 32-bit division, and on
// the scalar unit when n is uniform.
struct FastDiv {
  uint32_t m, k;
  static FastDiv of(long d) {
    uint32_t s = 0;
    while ((1L << s) < d) s++;
    FastDiv f;
    f.k = 31 + s;
    const unsigned __int128 p = (unsigned __int128)1 << f.k;
    f.m = (uint32_t)(p / (unsigned long)d + (p % (unsigned long)d ? 1 : 0));
    return f;
  }
  __host__ __device__ __forceinline__ uint32_t div(uint32_t n) const {
    return (uint32_t)(((uint64_t)n * m) >> k);
  }
};

// The weight of one synapse from its traces, shared by the trace/weight kernel and the rewiring
// kernels so both see bit-identical values:  log(max(cij, cthr^4) / (ci * cj)) evaluated as
// log(max(cij, cthr^4) * (1/ci) * (1/cj)).  rci / rcj are the reciprocals, or a negative number when
// the row / column trace is below cthr (the weight is then zero).
template <typename T>
__device__ __forceinline__ T trace_reciprocal(T c, T cthr) {
  return (c < cthr) ? T(-1) : Real<T>::div(T(1), c);
}
template <typename T>
__device__ __forceinline__ T weight_from_traces(T cij, T rci, T rcj, T cthr4) {
  const T num = fmax(cij, cthr4);  // cthr4 as well when cij is NaN, like `cij > cthr4 ? cij : cthr4`
  const T w = Real<T>::wlog(num * rci * rcj);
  return (rci < T(0) || rcj < T(0)) ? T(0) : w;
}

}  // namespace sb
