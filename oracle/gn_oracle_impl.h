/* Body of the CPU oracle, included once per arithmetic type (REAL = double, float).
 * TEST INFRASTRUCTURE ONLY -- see gn_oracle.c. */

#define FN2(name, suf) name##_##suf
#define FN1(name, suf) FN2(name, suf)
#define FN(name) FN1(name, SUF)

/* Activations and derivatives: src/gnnhwc/csrc/gn_kernel.cu:62-106. */
static REAL FN(act)(REAL x, int act) {
  switch (act) {
    case 0: return x;                                                   /* identity   :62 */
    case 1: return x > 0 ? x : (REAL)0;                                 /* relu       :64 */
    case 2: return x / ((REAL)1 + (REAL)exp(-(double)x));               /* silu       :66 */
    case 3: return x * (REAL)0.5 * ((REAL)1 + (REAL)erf((double)x * M_SQRT1_2)); /* gelu :71-74 */
    default: {                                                          /* gelu_tanh  :83-88 */
      const REAL kBeta = (REAL)(M_SQRT2 * M_2_SQRTPI * 0.5);
      const REAL inner = kBeta * (x + (REAL)0.044715 * x * x * x);
      return (REAL)0.5 * x * ((REAL)1 + (REAL)tanh((double)inner));
    }
  }
}
static REAL FN(act_d)(REAL x, int act) {
  switch (act) {
    case 0: return (REAL)1;                                             /* :63 */
    case 1: return x > 0 ? (REAL)1 : (REAL)0;                           /* :65 */
    case 2: {                                                           /* :67-70 */
      const REAL s = (REAL)1 / ((REAL)1 + (REAL)exp(-(double)x));
      return s * ((REAL)1 + x * ((REAL)1 - s));
    }
    case 3: {                                                           /* :75-82 */
      const REAL cdf = (REAL)0.5 * ((REAL)1 + (REAL)erf((double)x * M_SQRT1_2));
      const REAL pdf = (REAL)exp(-0.5 * (double)x * (double)x) * (REAL)(M_2_SQRTPI * M_SQRT1_2 * 0.5);
      return cdf + x * pdf;
    }
    default: {                                                          /* :89-106 */
      const REAL kBeta = (REAL)(M_SQRT2 * M_2_SQRTPI * 0.5);
      const REAL kKappa = (REAL)0.044715;
      const REAL x_sq = x * x;
      const REAL inner = kBeta * (x + kKappa * x_sq * x);
      const REAL t = (REAL)tanh((double)inner);
      const REAL left_derivative = (REAL)0.5 * ((REAL)1 + t);
      const REAL right_derivative = (REAL)0.5 * x * ((REAL)1 - t * t) * kBeta * ((REAL)1 + (REAL)3 * kKappa * x_sq);
      return left_derivative + right_derivative;
    }
  }
}

/* Per-(n, g) statistics with the reference's streaming update:
 *   WelfordOps::reduce  (src/gnnhwc/csrc/Welford.h:30-42): delta = x - mean; mean += delta / n; m2 += delta * (x - mean)
 *   WelfordOps::project (Welford.h:66-72) with correction 0 (gn_kernel.cu:175,254): var = m2 / n
 *   rstd = rsqrt(var + eps) (gn_kernel.cu:290-291)
 * x is (N, R, C) with C fastest (custom_gn.cpp:24). */
void FN(gn_oracle_stats)(const REAL *x, int64_t N, int64_t R, int64_t C, int64_t G, double eps, REAL *mean, REAL *rstd) {
  const int64_t D = C / G;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    for (int64_t g = 0; g < G; ++g) {
      REAL mu = 0, m2 = 0, cnt = 0;
      for (int64_t r = 0; r < R; ++r) {
        const REAL *row = x + (n * R + r) * C + g * D;
        for (int64_t d = 0; d < D; ++d) {
          const REAL v = row[d];
          const REAL delta = v - mu;
          cnt += 1;
          mu += delta / cnt;
          m2 += delta * (v - mu);
        }
      }
      mean[n * G + g] = mu;
      rstd[n * G + g] = (REAL)1 / (REAL)sqrt((double)(m2 / cnt + (REAL)eps));
    }
  }
}

/* Forward: a = rstd * gamma, b = -mean * a + beta, y = act(x * a + b)
 * (scale_shift_kernel, gn_kernel.cu:350-379 and :396-409). */
void FN(gn_oracle_fwd)(const REAL *x, const REAL *w, const REAL *b, int64_t N, int64_t R, int64_t C, int64_t G,
                       double eps, int act, REAL *y, REAL *mean, REAL *rstd) {
  const int64_t D = C / G;
  FN(gn_oracle_stats)(x, N, R, C, G, eps, mean, rstd);
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    for (int64_t r = 0; r < R; ++r) {
      const REAL *xr = x + (n * R + r) * C;
      REAL *yr = y + (n * R + r) * C;
      for (int64_t c = 0; c < C; ++c) {
        const int64_t g = c / D;
        const REAL a = rstd[n * G + g] * w[c];
        const REAL s = -mean[n * G + g] * a + b[c];
        yr[c] = FN(act)(xr[c] * a + s, act);
      }
    }
  }
}

/* Backward.
 *   S1[n,c] = sum_r dy act'(z) x, S2[n,c] = sum_r dy act'(z), z = x a + b   (width_reduce, gn_kernel.cu:598-618)
 *   dgamma[c] = sum_n (S1 - mean S2) rstd, dbeta[c] = sum_n S2                 (compute_dweight_dbias, :717-727)
 *   A[n,g] = sum_{c in g} gamma S1, B[n,g] = sum_{c in g} gamma S2, s = 1/(D R)
 *   coef1 = (mean B - A) s rstd^3, coef2 = -mean coef1 - B s rstd               (compute_bwd_scale_biases, :783-800)
 *   dx = a dy act'(z) + coef1 x + coef2                                        (dx_elem_kernel, :868-871)
 * Same algebra as GN_Naive.bwd (test/check_outputs.py:34-48).  scratch: 2 N C REALs. */
void FN(gn_oracle_bwd)(const REAL *dy, const REAL *x, const REAL *w, const REAL *b, const REAL *mean, const REAL *rstd,
                       int64_t N, int64_t R, int64_t C, int64_t G, int act, REAL *dx, REAL *dw, REAL *db,
                       REAL *scratch) {
  const int64_t D = C / G;
  REAL *S1 = scratch, *S2 = scratch + N * C;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    for (int64_t g = 0; g < G; ++g) {
      for (int64_t d = 0; d < D; ++d) {
        const int64_t c = g * D + d;
        const REAL a = rstd[n * G + g] * w[c];
        const REAL s = -mean[n * G + g] * a + b[c];
        REAL t1 = 0, t2 = 0;
        for (int64_t r = 0; r < R; ++r) {
          const int64_t i = (n * R + r) * C + c;
          const REAL gd = dy[i] * FN(act_d)(x[i] * a + s, act);
          t1 += gd * x[i];
          t2 += gd;
        }
        S1[n * C + c] = t1;
        S2[n * C + c] = t2;
      }
    }
  }
  for (int64_t c = 0; c < C; ++c) {
    const int64_t g = c / D;
    REAL t1 = 0, t2 = 0;
    for (int64_t n = 0; n < N; ++n) {
      t1 += (S1[n * C + c] - mean[n * G + g] * S2[n * C + c]) * rstd[n * G + g];
      t2 += S2[n * C + c];
    }
    dw[c] = t1;
    db[c] = t2;
  }
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    for (int64_t g = 0; g < G; ++g) {
      const REAL mu = mean[n * G + g], rs = rstd[n * G + g];
      REAL A = 0, B = 0;
      for (int64_t d = 0; d < D; ++d) {
        const int64_t c = g * D + d;
        A += w[c] * S1[n * C + c];
        B += w[c] * S2[n * C + c];
      }
      const REAL s = (REAL)1 / (REAL)(D * R);
      const REAL coef1 = (mu * B - A) * s * rs * rs * rs;
      const REAL coef2 = -mu * coef1 - B * s * rs;
      for (int64_t r = 0; r < R; ++r) {
        for (int64_t d = 0; d < D; ++d) {
          const int64_t c = g * D + d;
          const int64_t i = (n * R + r) * C + c;
          const REAL a = rs * w[c];
          const REAL sh = -mu * a + b[c];
          dx[i] = a * dy[i] * FN(act_d)(x[i] * a + sh, act) + coef1 * x[i] + coef2;
        }
      }
    }
  }
}

#undef FN
#undef FN1
#undef FN2
