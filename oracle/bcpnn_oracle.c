/*
 * TEST INFRASTRUCTURE ONLY.  Nothing the product ships may link, load or call this file; it is the
 * checker that the GPU parity tests, the smoke test and the bench's cpu_baseline leg compare against.
 *
 * Plain-C restatement of the StreamBrain cpu (OpenMP) backend's per-batch kernels
 * (BCPNN/backend/_kernels/kernels_openmp_internal.cc and the numpy softmax the cpu backend binds,
 * BCPNN/backend/_kernels/kernels_numpy.py:13-25), in float and double.
 *
 * Build variants (see build.py next to this file):
 *   libbcpnn_oracle.so       strict IEEE: -O2 -ffp-contract=off, the arithmetic order written here
 *   libbcpnn_oracle_fast.so  -O3 -march=x86-64-v3 -ffast-math -fopenmp, the reference's own flag set
 *                            (CMakeLists.txt:18-24,39-40) -- used as the timed CPU baseline and to
 *                            bound the fast-math spread.
 *
 * Pinning status (what fixes each function independently of this restatement) is listed in
 * oracle/README.md and exercised by tests/test_oracle_pins.py.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_CAT_(a, b) a##b
#define ORACLE_CAT(a, b) ORACLE_CAT_(a, b)

#define REAL float
#define FN(name) ORACLE_CAT(name, _f32)
#define LOG logf
#define EXP expf
#define ORACLE_LANES 16 /* 64-byte vectors of float, omp.cc:8-10,95-96 */
#include "bcpnn_oracle_impl.h"
#undef REAL
#undef FN
#undef LOG
#undef EXP
#undef ORACLE_LANES

#define REAL double
#define FN(name) ORACLE_CAT(name, _f64)
#define LOG log
#define EXP exp
#define ORACLE_LANES 8
#include "bcpnn_oracle_impl.h"
#undef REAL
#undef FN
#undef LOG
#undef EXP
#undef ORACLE_LANES

int oracle_abi_version(void) { return 1; }
