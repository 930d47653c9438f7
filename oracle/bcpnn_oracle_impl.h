/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the StreamBrain cpu (OpenMP) backend kernels.
 *
 * This body is included twice by bcpnn_oracle.c, once with REAL=float (suffix _f32) and once with
 * REAL=double (suffix _f64).  Each function names the reference lines whose arithmetic order it
 * restates; paths are relative to the reference checkout
 * (BCPNN/backend/_kernels/kernels_openmp_internal.cc is abbreviated "omp.cc").
 *
 * All matrices are dense row-major: x[B,N], y[B,M], W[N,M], Cij[N,M], wmask[N,H] (uint8).
 */

/* omp.cc:70-87 (matmul_add_bias) on top of omp.cc:40-61 (row-major NN gemm, alpha=1, beta=0).
 * The BLAS accumulation order is vendor-defined; this restatement accumulates k = 0..N-1 in REAL. */
void FN(oracle_update_state)(REAL *act, const REAL *x, const REAL *W, const REAL *bias,
                             long B, long N, long M) {
#pragma omp parallel for schedule(static)
  for (long b = 0; b < B; b++) {
    REAL *row = act + b * M;
    for (long j = 0; j < M; j++) row[j] = (REAL)0;
    for (long k = 0; k < N; k++) {
      const REAL a = x[b * N + k];
      const REAL *w = W + k * M;
      for (long j = 0; j < M; j++) row[j] += a * w[j];
    }
    for (long j = 0; j < M; j++) row[j] += bias[j];
  }
}

/* kernels_numpy.py:13-25 (softmax over the minicolumns of each hypercolumn), bound to the cpu
 * backend at cpu_backend.py:10,24.  t = exp(x - max); t / sum(t), per (sample, hypercolumn). */
void FN(oracle_softmax_minicolumns)(REAL *act, long B, long H, long Mc) {
#pragma omp parallel for schedule(static)
  for (long g = 0; g < B * H; g++) {
    REAL *v = act + g * Mc;
    REAL mx = v[0];
    for (long c = 1; c < Mc; c++) mx = v[c] > mx ? v[c] : mx;
    REAL s = (REAL)0;
    for (long c = 0; c < Mc; c++) {
      v[c] = EXP(v[c] - mx);
      s += v[c];
    }
    for (long c = 0; c < Mc; c++) v[c] = v[c] / s;
  }
}

/* omp.cc:89-205 (vectorized_updateWeights): Ci / Cj / Cij moving averages with clamp at zero and the
 * weight recompute from the freshly stored traces.  Per output lane the batch sum runs b = 0..B-1 in
 * REAL (omp.cc:109-115,135-141,167-176), then /B, then *taupdt, then C*(1-taupdt)+tmp, then max(0,.)
 * (omp.cc:117-129,143-155,178-190).  (1-taupdt) is formed in double and narrowed (omp.cc:101);
 * cthr^4 is formed in REAL by repeated multiplication (omp.cc:102).  Returns the scalar C of
 * omp.cc:98-99 (callers ignore it, kernels_openmp.py:18-25). */
REAL FN(oracle_update_weights)(REAL C, REAL *Ci, REAL *Cj, REAL *Cij, const REAL *a_i,
                               const REAL *a_o, REAL taupdt, long B, long N, long M, REAL *W,
                               REAL cthr) {
  C = (1 - taupdt) * C + taupdt;
  C = C > (REAL)0 ? C : (REAL)0;
  const REAL omt = (REAL)(1.0 - (double)taupdt);
  const REAL cthr4 = cthr * cthr * cthr * cthr;
  const REAL fB = (REAL)B;

#pragma omp parallel
  {
#pragma omp for schedule(static) nowait
    for (long i = 0; i < N; i++) { /* omp.cc:106-130 */
      REAL tmp = (REAL)0;
      for (long b = 0; b < B; b++) tmp += a_i[b * N + i];
      tmp /= fB;
      tmp *= taupdt;
      REAL c = Ci[i] * omt;
      c += tmp;
      Ci[i] = c > (REAL)0 ? c : (REAL)0;
    }
#pragma omp for schedule(static)
    for (long j = 0; j < M; j++) { /* omp.cc:132-156 */
      REAL tmp = (REAL)0;
      for (long b = 0; b < B; b++) tmp += a_o[b * M + j];
      tmp /= fB;
      tmp *= taupdt;
      REAL c = Cj[j] * omt;
      c += tmp;
      Cj[j] = c > (REAL)0 ? c : (REAL)0;
    }
#pragma omp for schedule(static)
    for (long i = 0; i < N; i++) { /* omp.cc:158-201 */
      const int skip = Ci[i] < cthr;
      REAL *wrow = W + i * M;
      REAL *crow = Cij + i * M;
      if (skip) memset(wrow, 0, sizeof(REAL) * (size_t)M); /* omp.cc:160-162 */
      for (long j0 = 0; j0 < M; j0 += ORACLE_LANES) {
        const long nl = (M - j0) < ORACLE_LANES ? (M - j0) : ORACLE_LANES;
        REAL tmp[ORACLE_LANES];
        for (long v = 0; v < nl; v++) tmp[v] = (REAL)0;
        for (long b = 0; b < B; b++) {
          const REAL a = a_i[b * N + i];
          const REAL *o = a_o + b * M + j0;
          for (long v = 0; v < nl; v++) tmp[v] += a * o[v];
        }
        for (long v = 0; v < nl; v++) {
          REAL t = tmp[v] / fB;
          t *= taupdt;
          REAL c = crow[j0 + v] * omt;
          c += t;
          c = c > (REAL)0 ? c : (REAL)0;
          crow[j0 + v] = c;
          if (!skip) { /* omp.cc:192-199 */
            const REAL cj = Cj[j0 + v];
            if (cj < cthr) {
              wrow[j0 + v] = (REAL)0;
            } else {
              const REAL num = c > cthr4 ? c : cthr4;
              wrow[j0 + v] = LOG(num / (Ci[i] * cj));
            }
          }
        }
      }
    }
  }
  return C;
}

/* omp.cc:207-220 (update_bias). */
void FN(oracle_update_bias)(REAL *bias, const REAL *Cj, REAL cthr, long M) {
  for (long j = 0; j < M; j++) {
    if (Cj[j] < cthr)
      bias[j] = LOG((REAL)2 * cthr);
    else
      bias[j] = LOG(Cj[j]);
  }
}

/* omp.cc:222-246 (update_bias_regularized). */
void FN(oracle_update_bias_regularized)(REAL *bias, REAL *kbi, const REAL *Cj, REAL cthr, REAL khalf,
                                        REAL pmin, REAL taubdt, long M) {
  const REAL p4 = pmin / (REAL)4;
  const REAL k = (khalf - 1) * (p4 * p4);
  for (long j = 0; j < M; j++) {
    const REAL pj = Cj[j];
    REAL kb = 1 + k / ((pj - p4) * (pj - p4));
    if (pj < p4 || kb < khalf) kb = khalf;
    kbi[j] = (1 - taubdt) * kbi[j] + taubdt * kb;
    if (Cj[j] < cthr)
      bias[j] = kbi[j] * LOG((REAL)2 * cthr);
    else
      bias[j] = kbi[j] * LOG(pj);
  }
}

/* omp.cc:248-320 (update_mask).  The score quotient is evaluated in double and narrowed, because the
 * reference writes nominator / (1.0 + (REAL)csum) (omp.cc:293).  Candidates are scanned in ascending
 * row order with >= / <=, so among equal scores the LAST row wins (omp.cc:294-304).
 * Optional trace output (each may be NULL): per executed swap, swaps[2*t..] = {imax0, imin1},
 * vals[2*t..] = {vmax0, vmin1} and runner[2*t..] = {the best score among the other silent rows, the worst
 * among the other active rows} at that iteration (the margins by which the two picks won; -3e38 / +3e38
 * when a side had one candidate only); *nswaps receives the number of swaps performed; stop[0..2] =
 * {1, vmax0, vmin1} when the loop ended by vmax0 < vmin1, {0, 0, 0} otherwise.  The trace changes nothing of
 * the result. */
void FN(oracle_update_mask)(uint8_t *wmask, const REAL *W, const REAL *Ci, const REAL *Cj,
                            const REAL *Cij, REAL cthr, long N, long M, long h, long H, long Mc,
                            long iterations, long *swaps, REAL *vals, long *nswaps, REAL *runner,
                            REAL *stop) {
  REAL *nom = (REAL *)calloc((size_t)N, sizeof(REAL));
  int *csum = (int *)calloc((size_t)N, sizeof(int));
#pragma omp parallel for schedule(static)
  for (long i = 0; i < N; i++) { /* omp.cc:257-277 */
    REAL score = (REAL)0;
    for (long j = h * Mc; j < (h + 1) * Mc; j++) {
      if (Ci[i] >= cthr && Cj[j] >= cthr) {
        const REAL pi = Ci[i];
        const REAL pj = Cj[j];
        const REAL pij = Cij[i * M + j];
        const REAL x = (1 - pi) * pj;
        const REAL y = (pj - pij) / x;
        const REAL WijC = LOG(y);
        score += pij * W[i * M + j] + (pj - pij) * WijC;
      }
    }
    nom[i] = score;
    int s = 0;
    for (long g = 0; g < H; g++) s += wmask[i * H + g]; /* omp.cc:279-287 */
    csum[i] = s;
  }
  long done = 0;
  for (long it = 0; it < iterations; it++) { /* omp.cc:289-315 */
    REAL vmax0 = (REAL)0, vmin1 = (REAL)0;
    long imax0 = N, imin1 = N;
    for (long j = 0; j < N; j++) {
      const REAL score = (REAL)((double)nom[j] / (1.0 + (double)(REAL)csum[j]));
      if (wmask[j * H + h] == 0 && (imax0 == N || score >= vmax0)) {
        imax0 = j;
        vmax0 = score;
      } else if (wmask[j * H + h] == 1 && (imin1 == N || score <= vmin1)) {
        imin1 = j;
        vmin1 = score;
      }
    }
    if (stop) {
      stop[0] = stop[1] = stop[2] = (REAL)0;
      if (imax0 != N && imin1 != N && vmax0 < vmin1) stop[0] = (REAL)1, stop[1] = vmax0, stop[2] = vmin1;
    }
    if (imax0 == N || imin1 == N || vmax0 < vmin1) break;
    if (runner) { /* second scan, trace only: the runners-up of this iteration */
      REAL r0 = (REAL)-3e38, r1 = (REAL)3e38;
      for (long j = 0; j < N; j++) {
        if (j == imax0 || j == imin1) continue;
        const REAL score = (REAL)((double)nom[j] / (1.0 + (double)(REAL)csum[j]));
        if (wmask[j * H + h] == 0 && score > r0) r0 = score;
        else if (wmask[j * H + h] == 1 && score < r1) r1 = score;
      }
      runner[2 * done] = r0;
      runner[2 * done + 1] = r1;
    }
    wmask[imax0 * H + h] = 1;
    wmask[imin1 * H + h] = 0;
    csum[imax0] += 1;
    csum[imin1] -= 1;
    if (swaps) {
      swaps[2 * done] = imax0;
      swaps[2 * done + 1] = imin1;
    }
    if (vals) {
      vals[2 * done] = vmax0;
      vals[2 * done + 1] = vmin1;
    }
    done++;
  }
  if (nswaps) *nswaps = done;
  free(csum);
  free(nom);
}

/* omp.cc:322-335 (apply_mask). */
void FN(oracle_apply_mask)(REAL *W, const uint8_t *wmask, long N, long M, long H, long Mc) {
#pragma omp parallel for schedule(static)
  for (long i = 0; i < N; i++) {
    for (long j = 0; j < M; j++) {
      const long h = j / Mc;
      if (!wmask[i * H + h]) W[i * M + j] = (REAL)0;
    }
  }
}

/* _cpu_base_backend.py:239-240: np.argmax(activations, axis=1) -- first maximal index per row. */
void FN(oracle_argmax_rows)(const REAL *act, long B, long M, int32_t *out) {
  for (long b = 0; b < B; b++) {
    long best = 0;
    for (long j = 1; j < M; j++)
      if (act[b * M + j] > act[b * M + best]) best = j;
    out[b] = (int32_t)best;
  }
}
