/*
 * rownorm_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A scalar CPU restatement (plain C, double accumulators) of the row-wise
 * reduce-then-normalize operators that intel/torch-xpu-ops implements in
 *   src/ATen/native/xpu/sycl/LayerNormKernels.cpp
 *   src/ATen/native/xpu/sycl/Norm.h
 *   src/ATen/native/xpu/sycl/SoftMaxKernels.cpp
 *   src/ATen/native/xpu/sycl/GroupNormKernels.cpp
 *   src/ATen/native/xpu/sycl/SharedReduceOps.h
 * It is the checker the GPU kernels are compared against.  Only the test
 * suite, the smoke check and the bench's CPU-baseline leg may load it; the
 * shipped library never does.
 *
 * The arithmetic parity target of those operators is PyTorch's CPU ATen
 * implementation (third-party, not vendored in the reference; torch 2.10.0
 * is the version installed beside this file's users).  The published
 * algorithms are restated here with every reduction carried in double, so
 * the oracle is the "fp32-accumulated-or-better" reference that low
 * precision results are compared with.
 *
 * Pinning (see tests/test_oracle_*.py): every function below is checked
 * against (1) committed torch-CPU golden vectors, (2) numpy/scipy closed
 * forms (mean/var, scipy.special.softmax/log_softmax), (3) central finite
 * differences of the forward functions for each backward function, and
 * (4) invariants (sum softmax = 1, sum softmax-backward = 0, dbeta of a
 * sum() loss = row count, constant row -> beta), (5) for the masked and
 * safe softmax variants, the plain functions applied to the unmasked
 * elements alone, (6) for GroupNorm, the LayerNorm functions applied to each
 * (sample, group) slab with the per-channel weights expanded per element.
 * No function is "parity unpinned".
 *
 * All arrays are dense row-major float32; low-precision inputs are passed
 * already widened to float32 (exactly representable), outputs are returned
 * unrounded in float32.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>

/* ------------------------------------------------------------------ */
/* Welford accumulator: SharedReduceOps.h:31-102 (WelfordData/WelfordOps) */
typedef struct {
  double mean, m2, nf;
} welford_t;

/* WelfordOps::reduce, SharedReduceOps.h:56-70 */
static welford_t welford_push(welford_t a, double x) {
  double nf = a.nf + 1.0;
  double delta = x - a.mean;
  double mean = a.mean + delta / nf;
  welford_t r = {mean, a.m2 + delta * (x - mean), nf};
  return r;
}

/* WelfordOps::combine (delta form), SharedReduceOps.h:71-88 */
static welford_t welford_merge(welford_t a, welford_t b) {
  if (a.nf == 0) return b;
  if (b.nf == 0) return a;
  double delta = b.mean - a.mean;
  double n = a.nf + b.nf;
  double nb_over_n = b.nf / n;
  welford_t r = {a.mean + delta * nb_over_n,
                 a.m2 + b.m2 + delta * delta * a.nf * nb_over_n, n};
  return r;
}

/* Row moments with a two-level Welford (chunks of 64 combined pairwise in
 * order), the shape the device kernels use: RowwiseMomentsFunctor,
 * LayerNormKernels.cpp:203-252 (biased variance: project() with correction 0,
 * SharedReduceOps.h:89-95). */
void oracle_welford_moments(const float* x, int64_t n, double* mean_out,
                            double* var_out) {
  welford_t total = {0, 0, 0};
  for (int64_t i = 0; i < n; i += 64) {
    welford_t c = {0, 0, 0};
    int64_t e = i + 64 < n ? i + 64 : n;
    for (int64_t j = i; j < e; ++j) c = welford_push(c, (double)x[j]);
    total = welford_merge(total, c);
  }
  *mean_out = total.mean;
  *var_out = total.nf > 0 ? total.m2 / total.nf : NAN;
}

/* ------------------------------------------------------------------ */
/* native_layer_norm forward.
 * Stats: LayerNormKernels.cpp:203-252 (rstd = rsqrt(var + eps), :222-230).
 * Normalize: y = gamma * (rstd * (x - mean)) + beta,
 * LayerNormKernels.cpp:274-320 and the vectorized form :494-542; a null
 * gamma/beta means 1/0 (:281-285). */
void oracle_layer_norm_fwd(const float* x, const float* gamma,
                           const float* beta, float* y, float* mean,
                           float* rstd, int64_t M, int64_t N, double eps) {
  for (int64_t r = 0; r < M; ++r) {
    const float* xr = x + r * N;
    double mu, var;
    oracle_welford_moments(xr, N, &mu, &var);
    if (var < 0) var = 0;
    double rs = 1.0 / sqrt(var + eps);
    if (mean) mean[r] = (float)mu;
    if (rstd) rstd[r] = (float)rs;
    if (y) {
      float* yr = y + r * N;
      for (int64_t j = 0; j < N; ++j) {
        double g = gamma ? (double)gamma[j] : 1.0;
        double b = beta ? (double)beta[j] : 0.0;
        yr[j] = (float)(g * (rs * ((double)xr[j] - mu)) + b);
      }
    }
  }
}

/* _fused_rms_norm forward: rstd = rsqrt(mean(x^2) + eps),
 * y = gamma * (rstd * x).  LayerNormKernels.cpp:227-229 (the rms branch of
 * the moments functor: m2 + m1^2 is E[x^2]) and :508-509. */
void oracle_rms_norm_fwd(const float* x, const float* gamma, float* y,
                         float* rstd, int64_t M, int64_t N, double eps) {
  for (int64_t r = 0; r < M; ++r) {
    const float* xr = x + r * N;
    double ss = 0;
    for (int64_t j = 0; j < N; ++j) ss += (double)xr[j] * (double)xr[j];
    double rs = 1.0 / sqrt(ss / (double)N + eps);
    if (rstd) rstd[r] = (float)rs;
    if (y) {
      float* yr = y + r * N;
      for (int64_t j = 0; j < N; ++j) {
        double g = gamma ? (double)gamma[j] : 1.0;
        yr[j] = (float)(g * (rs * (double)xr[j]));
      }
    }
  }
}

/* native_layer_norm_backward.
 * dX: LayerNormBackward::reduce_combine/update, LayerNormKernels.cpp:86-186:
 *   s1 = sum dy*gamma, s2 = sum dy*gamma*(x-mean)*rstd,
 *   dx = (rstd/N) * (N*gamma*dy - (x-mean)*rstd*s2 - s1).
 * dgamma/dbeta: GammaBetaBackwardSimpleKernelFunctor,
 * LayerNormKernels.cpp:885-1024 (:901-934):
 *   dgamma[j] = sum_i dy*(x-mean_i)*rstd_i, dbeta[j] = sum_i dy.
 * Any of dx/dgamma/dbeta may be NULL (skipped, :1140,1270-1406). */
void oracle_layer_norm_bwd(const float* dy, const float* x, const float* mean,
                           const float* rstd, const float* gamma, float* dx,
                           float* dgamma, float* dbeta, double* col_scratch,
                           int64_t M, int64_t N) {
  /* col_scratch: 2*N doubles for the column sums */
  double* dg = col_scratch;
  double* db = col_scratch + N;
  for (int64_t j = 0; j < 2 * N; ++j) col_scratch[j] = 0;
  for (int64_t r = 0; r < M; ++r) {
    const float* xr = x + r * N;
    const float* gr = dy + r * N;
    double mu = (double)mean[r], rs = (double)rstd[r];
    double s1 = 0, s2 = 0;
    for (int64_t j = 0; j < N; ++j) {
      double g = gamma ? (double)gamma[j] : 1.0;
      double v = (double)gr[j] * g;
      double xhat = ((double)xr[j] - mu) * rs;
      s1 += v;
      s2 += v * xhat;
      dg[j] += (double)gr[j] * xhat;
      db[j] += (double)gr[j];
    }
    if (dx) {
      float* dr = dx + r * N;
      double term1 = rs / (double)N;
      for (int64_t j = 0; j < N; ++j) {
        double g = gamma ? (double)gamma[j] : 1.0;
        double f = (double)N * g * (double)gr[j];
        f -= ((double)xr[j] - mu) * rs * s2;
        f -= s1;
        dr[j] = (float)(f * term1);
      }
    }
  }
  if (dgamma)
    for (int64_t j = 0; j < N; ++j) dgamma[j] = (float)dg[j];
  if (dbeta)
    for (int64_t j = 0; j < N; ++j) dbeta[j] = (float)db[j];
}

/* _fused_rms_norm_backward: the rms_norm branches of the same functors
 * (LayerNormKernels.cpp:118-122, 176-178, 925-927):
 *   s2 = sum dy*gamma*x*rstd, dx = (rstd/N) * (N*gamma*dy - x*rstd*s2),
 *   dgamma[j] = sum_i dy*x*rstd_i. */
void oracle_rms_norm_bwd(const float* dy, const float* x, const float* rstd,
                         const float* gamma, float* dx, float* dgamma,
                         double* col_scratch, int64_t M, int64_t N) {
  double* dg = col_scratch; /* N doubles */
  for (int64_t j = 0; j < N; ++j) dg[j] = 0;
  for (int64_t r = 0; r < M; ++r) {
    const float* xr = x + r * N;
    const float* gr = dy + r * N;
    double rs = (double)rstd[r];
    double s2 = 0;
    for (int64_t j = 0; j < N; ++j) {
      double g = gamma ? (double)gamma[j] : 1.0;
      double xhat = (double)xr[j] * rs;
      s2 += (double)gr[j] * g * xhat;
      dg[j] += (double)gr[j] * xhat;
    }
    if (dx) {
      float* dr = dx + r * N;
      double term1 = rs / (double)N;
      for (int64_t j = 0; j < N; ++j) {
        double g = gamma ? (double)gamma[j] : 1.0;
        double f = (double)N * g * (double)gr[j] - (double)xr[j] * rs * s2;
        dr[j] = (float)(f * term1);
      }
    }
  }
  if (dgamma)
    for (int64_t j = 0; j < N; ++j) dgamma[j] = (float)dg[j];
}

/* _softmax / _log_softmax over the last dimension.
 * DispatchSoftmaxForwardKernelFunctor, SoftMaxKernels.cpp:212-410:
 *   m = max x; s = sum exp(x - m); softmax = exp(x-m)/s;
 *   log_softmax = x - m - log s.  A row with no finite maximum (all -inf)
 *   gives NaN, as x - m is NaN (and :331-332 maps s == 0 to NaN). */
void oracle_softmax_fwd(const float* x, float* y, int64_t rows, int64_t N,
                        int is_log) {
  for (int64_t r = 0; r < rows; ++r) {
    const float* xr = x + r * N;
    float* yr = y + r * N;
    double m = -INFINITY;
    int has_nan = 0;
    for (int64_t j = 0; j < N; ++j) {
      if (xr[j] != xr[j]) has_nan = 1;
      if ((double)xr[j] > m) m = (double)xr[j];
    }
    if (has_nan) m = NAN;
    double s = 0;
    for (int64_t j = 0; j < N; ++j) s += exp((double)xr[j] - m);
    if (is_log) {
      double ls = log(s);
      for (int64_t j = 0; j < N; ++j) yr[j] = (float)((double)xr[j] - m - ls);
    } else {
      for (int64_t j = 0; j < N; ++j)
        yr[j] = (float)(exp((double)xr[j] - m) / s);
    }
  }
}

/* _softmax_backward_data / _log_softmax_backward_data.
 * DispatchSoftmaxBackwardKernelFunctor, SoftMaxKernels.cpp:952-1102
 * (:1031-1047): softmax gi = y*(g - sum y*g); log_softmax
 * gi = g - exp(y)*sum g. */
void oracle_softmax_bwd(const float* g, const float* y, float* gi,
                        int64_t rows, int64_t N, int is_log) {
  for (int64_t r = 0; r < rows; ++r) {
    const float* gr = g + r * N;
    const float* yr = y + r * N;
    float* o = gi + r * N;
    double s = 0;
    if (is_log) {
      for (int64_t j = 0; j < N; ++j) s += (double)gr[j];
      for (int64_t j = 0; j < N; ++j)
        o[j] = (float)((double)gr[j] - exp((double)yr[j]) * s);
    } else {
      for (int64_t j = 0; j < N; ++j) s += (double)yr[j] * (double)gr[j];
      for (int64_t j = 0; j < N; ++j)
        o[j] = (float)((double)yr[j] * ((double)gr[j] - s));
    }
  }
}

/* _safe_softmax: softmax whose rows with no finite element come out as zeros.
 * is_safe_softmax branches, SoftMaxKernels.cpp:328-346 (max == -inf -> 0). */
void oracle_safe_softmax_fwd(const float* x, float* y, int64_t rows, int64_t N) {
  oracle_softmax_fwd(x, y, rows, N, 0);
  for (int64_t r = 0; r < rows; ++r) {
    int all_ninf = 1;
    for (int64_t j = 0; j < N; ++j)
      if (!(x[r * N + j] == -INFINITY)) all_ninf = 0;
    if (all_ninf)
      for (int64_t j = 0; j < N; ++j) y[r * N + j] = 0.0f;
  }
}

/* _masked_softmax over the last dimension; mask is [rows, N] bytes, non-zero
 * = leave the element out.  SoftMaxKernels.cpp:257-272 replaces masked
 * elements by -inf before the max; :331-332 turns a zero sum (every element
 * masked, or -inf wherever the mask leaves one in) into a NaN row. */
void oracle_masked_softmax_fwd(const float* x, const uint8_t* mask, float* y,
                               int64_t rows, int64_t N) {
  for (int64_t r = 0; r < rows; ++r) {
    const float* xr = x + r * N;
    const uint8_t* mr = mask + r * N;
    float* yr = y + r * N;
    double m = -INFINITY;
    int has_nan = 0, any = 0;
    for (int64_t j = 0; j < N; ++j) {
      if (mr[j]) continue;
      any = 1;
      if (xr[j] != xr[j]) has_nan = 1;
      if ((double)xr[j] > m) m = (double)xr[j];
    }
    if (has_nan) m = NAN;
    double s = 0;
    for (int64_t j = 0; j < N; ++j)
      if (!mr[j]) s += exp((double)xr[j] - m);
    for (int64_t j = 0; j < N; ++j) {
      if (!any || s == 0 || m == -INFINITY)
        yr[j] = NAN;
      else
        yr[j] = mr[j] ? 0.0f : (float)(exp((double)xr[j] - m) / s);
    }
  }
}

/* _masked_softmax_backward: softmax backward with the saved output read as 0
 * at masked positions (SoftMaxKernels.cpp:991-1001), hence gi = 0 * (g - s)
 * there: 0, or NaN when the row's unmasked outputs hold a NaN. */
void oracle_masked_softmax_bwd(const float* g, const float* y,
                               const uint8_t* mask, float* gi, int64_t rows,
                               int64_t N) {
  for (int64_t r = 0; r < rows; ++r) {
    const float* gr = g + r * N;
    const float* yr = y + r * N;
    const uint8_t* mr = mask + r * N;
    float* o = gi + r * N;
    double s = 0;
    for (int64_t j = 0; j < N; ++j)
      if (!mr[j]) s += (double)yr[j] * (double)gr[j];
    for (int64_t j = 0; j < N; ++j)
      o[j] = (float)((mr[j] ? 0.0 : (double)yr[j]) * ((double)gr[j] - s));
  }
}

/* native_group_norm on NCHW-contiguous [N, C, HxW] with G groups of D = C/G
 * channels.  GroupNormKernels.cpp:72-133 (row moments over the D*HxW elements
 * of a group, biased variance, rstd = 1/sqrt(var + eps)) and :220-260, :351-357
 * (y = x*a + b with a = rstd*gamma[c], b = beta[c] - a*mean).  mean/rstd are
 * [N, G]; gamma/beta may be NULL. */
void oracle_group_norm_fwd(const float* x, const float* gamma,
                           const float* beta, float* y, float* mean,
                           float* rstd, int64_t N, int64_t C, int64_t HxW,
                           int64_t G, double eps) {
  const int64_t D = G ? C / G : 0;
  const int64_t L = D * HxW;
  for (int64_t r = 0; r < N * G; ++r) {
    const float* xr = x + r * L;
    double mu, var;
    oracle_welford_moments(xr, L, &mu, &var);
    const double rs = 1.0 / sqrt(var + eps);
    if (mean) mean[r] = (float)mu;
    if (rstd) rstd[r] = (float)rs;
    const int64_t g = r % G;
    for (int64_t p = 0; p < L; ++p) {
      const int64_t c = g * D + p / HxW;
      const double a = rs * (gamma ? (double)gamma[c] : 1.0);
      const double b = (beta ? (double)beta[c] : 0.0) - a * mu;
      y[r * L + p] = (float)((double)xr[p] * a + b);
    }
  }
}

/* native_group_norm_backward, in the reference's own form:
 * ds[n,c] = sum_hw dy*x, db[n,c] = sum_hw dy (GroupNormKernels.cpp:955-975);
 * per (n,g): ds_sum = sum_c ds*gamma, db_sum = sum_c db*gamma,
 * c2 = (db_sum*mean - ds_sum)*rstd^3/(D*HxW), c3 = -c2*mean - db_sum*rstd/(D*HxW),
 * dx = rstd*gamma[c]*dy + c2*x + c3 (:1133-1160, :1081-1086);
 * dgamma[c] = sum_n (ds - db*mean)*rstd, dbeta[c] = sum_n db (:1195-1215).
 * mean/rstd are the saved [N, G] statistics.  Any output may be NULL. */
void oracle_group_norm_bwd(const float* dy, const float* x, const float* mean,
                           const float* rstd, const float* gamma, float* dx,
                           float* dgamma, float* dbeta, int64_t N, int64_t C,
                           int64_t HxW, int64_t G) {
  const int64_t D = G ? C / G : 0;
  const int64_t L = D * HxW;
  for (int64_t c = 0; c < C; ++c) {
    if (dgamma) dgamma[c] = 0;
    if (dbeta) dbeta[c] = 0;
  }
  if (N == 0 || L == 0) return;
  double* dgs = (double*)calloc((size_t)C, sizeof(double));
  double* dbs = (double*)calloc((size_t)C, sizeof(double));
  double* ds = (double*)malloc((size_t)(D ? D : 1) * sizeof(double));
  double* db = (double*)malloc((size_t)(D ? D : 1) * sizeof(double));
  for (int64_t r = 0; r < N * G; ++r) {
    const int64_t g = r % G;
    const double mu = mean[r], rs = rstd[r];
    double ds_sum = 0, db_sum = 0;
    for (int64_t d = 0; d < D; ++d) {
      double a = 0, b = 0;
      for (int64_t h = 0; h < HxW; ++h) {
        const int64_t i = r * L + d * HxW + h;
        a += (double)dy[i] * (double)x[i];
        b += (double)dy[i];
      }
      ds[d] = a;
      db[d] = b;
      const double ga = gamma ? (double)gamma[g * D + d] : 1.0;
      ds_sum += a * ga;
      db_sum += b * ga;
      dgs[g * D + d] += (a - b * mu) * rs;
      dbs[g * D + d] += b;
    }
    if (dx) {
      const double s = 1.0 / (double)L;
      const double c2 = (db_sum * mu - ds_sum) * rs * rs * rs * s;
      const double c3 = -c2 * mu - db_sum * rs * s;
      for (int64_t d = 0; d < D; ++d) {
        const double c1 = rs * (gamma ? (double)gamma[g * D + d] : 1.0);
        for (int64_t h = 0; h < HxW; ++h) {
          const int64_t i = r * L + d * HxW + h;
          dx[i] = (float)(c1 * (double)dy[i] + c2 * (double)x[i] + c3);
        }
      }
    }
  }
  for (int64_t c = 0; c < C; ++c) {
    if (dgamma) dgamma[c] = (float)dgs[c];
    if (dbeta) dbeta[c] = (float)dbs[c];
  }
  free(dgs);
  free(dbs);
  free(ds);
  free(db);
}
