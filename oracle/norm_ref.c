/*
 * norm_ref.c - plain C restatement of the reference's normalization
 * arithmetic (TEST INFRASTRUCTURE / CPU BASELINE ONLY, never linked into the
 * product).  float32 tensors in and out, double accumulators, loops in the
 * order the reference kernels reduce: per channel for BatchNormalization, per
 * row (Welford update + merge) for Layer/Group/InstanceNormalization.
 * OpenMP parallelises over channels / rows when built with -fopenmp; with
 * OMP_NUM_THREADS=1 it is the scalar port.
 *
 * Checked against oracle/norm_ref.py (which is pinned against torch float64
 * autograd) in tests/test_oracle_c.py.
 *
 * Citations are file:line under sony/nnabla-ext-cuda.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define NR_EXPORT __attribute__((visibility("default")))

NR_EXPORT int nr_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* n >= 1: threads of the following calls (1 = the scalar port). */
NR_EXPORT void nr_set_num_threads(int n) {
#ifdef _OPENMP
  if (n >= 1) omp_set_num_threads(n);
#else
  (void)n;
#endif
}

/* ---- Welford, include/nbla/cuda/utils/reduce_ops/welford.cuh:62-97 ------ */
typedef struct {
  double mean, m2;
  int64_t n;
} welford_t;

static inline void welford_update(welford_t *w, double x) {
  const double d = x - w->mean;           /* :63 */
  const double nm = w->mean + d / (double)(w->n + 1); /* :64 */
  w->m2 += d * (x - nm);                  /* :65 */
  w->mean = nm;
  w->n += 1;
}

static inline void welford_merge(welford_t *to, const welford_t *from) {
  if (to->n == 0) { *to = *from; return; }     /* :81-84 */
  if (from->n == 0) return;                    /* :85-87 */
  const int64_t n = to->n + from->n;
  const double inv = 1.0 / (double)n;
  const double d = from->mean - to->mean;
  to->mean += d * (double)from->n * inv;       /* :91 */
  to->m2 += from->m2 + d * d * (double)to->n * (double)from->n * inv; /* :92-93 */
  to->n = n;
}

/* Row statistics the way reduce_2d_x<WelfordOp> walks a row
 * (kernel/normalization.cuh:22-65): 8 interleaved partial states merged at the
 * end; variance = m2 / R (welford.cuh:100-103). */
static void row_stats(const float *x, int64_t R, double *mean, double *var) {
  welford_t part[8];
  for (int k = 0; k < 8; ++k) { part[k].mean = 0; part[k].m2 = 0; part[k].n = 0; }
  for (int64_t i = 0; i < R; ++i) welford_update(&part[i & 7], (double)x[i]);
  welford_t tot = part[0];
  for (int k = 1; k < 8; ++k) welford_merge(&tot, &part[k]);
  *mean = tot.mean;
  *var = tot.m2 / (double)R;
}

/* ---- BatchNormalization, x[size0][C][size2] ----------------------------- */

/* forward_global_kernel, kernel/batch_normalization.cuh:332-349 */
NR_EXPORT void nr_bn_forward_global(const float *x, const float *beta, const float *gamma,
                                    const float *rmean, const float *rvar, float *y,
                                    int64_t size0, int64_t C, int64_t size2, float eps) {
#pragma omp parallel for schedule(static)
  for (int64_t c = 0; c < C; ++c) {
    const double m = rmean[c];
    const double sd = sqrt((double)rvar[c] + eps);
    const double g = gamma ? gamma[c] : 1.0;
    const double b = beta ? beta[c] : 0.0;
    for (int64_t n = 0; n < size0; ++n) {
      const size_t base = ((size_t)n * C + c) * size2;
      for (int64_t i = 0; i < size2; ++i) y[base + i] = (float)(((double)x[base + i] - m) * g / sd + b);
    }
  }
}

/* forward_batch_* kernels, kernel/batch_normalization.cuh:259-325: sum and
 * sum of squares per channel, var = E[x^2]-mean^2 (biased), running stats with
 * N/(N-1) on the variance. */
NR_EXPORT void nr_bn_forward_batch(const float *x, const float *beta, const float *gamma,
                                   float *rmean, float *rvar, float *y, float *mean, float *var,
                                   int64_t size0, int64_t C, int64_t size2, float decay,
                                   float eps) {
  const double N = (double)size0 * (double)size2;
#pragma omp parallel for schedule(static)
  for (int64_t c = 0; c < C; ++c) {
    double s = 0, sq = 0;
    for (int64_t n = 0; n < size0; ++n) {
      const size_t base = ((size_t)n * C + c) * size2;
      for (int64_t i = 0; i < size2; ++i) {
        const double v = x[base + i];
        s += v;      /* :267 */
        sq += v * v; /* :268 */
      }
    }
    const double m = s / N;               /* :292 */
    const double v = sq / N - m * m;      /* :293 */
    mean[c] = (float)m;
    var[c] = (float)v;
    if (rmean) rmean[c] = (float)(decay * rmean[c] + (1.0 - decay) * m);            /* :296-298 */
    if (rvar) rvar[c] = (float)(decay * rvar[c] + (1.0 - decay) * v * (N / (N - 1.0))); /* :299-302 */
    const double inv = 1.0 / sqrt(v + eps); /* :319 */
    const double g = gamma ? gamma[c] : 1.0;
    const double b = beta ? beta[c] : 0.0;
    for (int64_t n = 0; n < size0; ++n) {
      const size_t base = ((size_t)n * C + c) * size2;
      for (int64_t i = 0; i < size2; ++i)
        y[base + i] = (float)(((double)x[base + i] - m) * g * inv + b); /* :323 */
    }
  }
}

/* backward_batch_* kernels, kernel/batch_normalization.cuh:402-469,502-540.
 * Gradients are written (not accumulated). dmean_in/dvar_in may be NULL. */
NR_EXPORT void nr_bn_backward_batch(const float *x, const float *dy, const float *gamma,
                                    const float *mean, const float *var, const float *dmean_in,
                                    const float *dvar_in, float *dx, float *dgamma, float *dbeta,
                                    int64_t size0, int64_t C, int64_t size2, float eps) {
  const double N = (double)size0 * (double)size2;
#pragma omp parallel for schedule(static)
  for (int64_t c = 0; c < C; ++c) {
    const double m = mean[c], v = var[c];
    const double g = gamma ? gamma[c] : 1.0;
    const double inv = 1.0 / sqrt(v + eps);
    double s_dyg = 0, s_dygx = 0, s_xc = 0, s_dy = 0, s_dyx = 0;
    for (int64_t n = 0; n < size0; ++n) {
      const size_t base = ((size_t)n * C + c) * size2;
      for (int64_t i = 0; i < size2; ++i) {
        const double d = dy[base + i];
        const double cx = (double)x[base + i] - m;
        s_dyg += d * g;        /* :413 */
        s_dygx += d * g * cx;  /* :412 */
        s_xc += cx;            /* :414 */
        s_dy += d;             /* :512 */
        s_dyx += d * cx;       /* :511 */
      }
    }
    const double dvar = s_dygx * -0.5 * pow(v + eps, -1.5) + (dvar_in ? dvar_in[c] : 0.0); /* :441-444 */
    const double dmean = s_dyg * -inv + dvar * -2.0 * s_xc / N + (dmean_in ? dmean_in[c] : 0.0); /* :446-448 */
    if (dgamma) dgamma[c] = (float)(s_dyx * inv);
    if (dbeta) dbeta[c] = (float)s_dy;
    if (dx) {
      for (int64_t n = 0; n < size0; ++n) {
        const size_t base = ((size_t)n * C + c) * size2;
        for (int64_t i = 0; i < size2; ++i) {
          const double cx = (double)x[base + i] - m;
          dx[base + i] = (float)((double)dy[base + i] * g * inv + dvar * 2.0 * cx / N + dmean / N); /* :464-466 */
        }
      }
    }
  }
}

/* ---- LayerNormalization, x[outer][R] ------------------------------------ */

/* reduce_2d_x<WelfordOp> + layer_norm_forward_normalization
 * (kernel/layer_normalization.cuh:24-48) */
NR_EXPORT void nr_ln_forward(const float *x, const float *beta, const float *gamma, float *y,
                             float *mean, float *var, int64_t outer, int64_t R, float eps) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < outer; ++r) {
    const float *xr = x + (size_t)r * R;
    float *yr = y + (size_t)r * R;
    double m, v;
    row_stats(xr, R, &m, &v);
    mean[r] = (float)m;
    var[r] = (float)v;
    const double inv = 1.0 / sqrt(v + eps);
    for (int64_t i = 0; i < R; ++i) {
      const double g = gamma ? gamma[i] : 1.0;
      const double b = beta ? beta[i] : 0.0;
      yr[i] = (float)(g * inv * ((double)xr[i] - m) + b); /* :45 */
    }
  }
}

/* LNGradOp + dx_factor + dx + dbeta_dgamma
 * (reduce_ops/layer_normalization.cuh:51-55, kernel/layer_normalization.cuh:50-120) */
NR_EXPORT void nr_ln_backward(const float *x, const float *dy, const float *gamma,
                              const float *mean, const float *var, const float *dmean,
                              const float *dvar, float *dx, float *dgamma, float *dbeta,
                              int64_t outer, int64_t R, float eps) {
  const double invR = 1.0 / (double)R;
  if (dx) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < outer; ++r) {
      const float *xr = x + (size_t)r * R;
      const float *dr = dy + (size_t)r * R;
      const double m = mean[r];
      const double inv = 1.0 / sqrt((double)var[r] + eps);
      double s1 = 0, s2 = 0;
      for (int64_t i = 0; i < R; ++i) {
        const double g = gamma ? gamma[i] : 1.0;
        s1 += dr[i] * g;                 /* sum_dygamma  */
        s2 += dr[i] * (double)xr[i] * g; /* sum_dyxgamma */
      }
      const double a = (s1 * m - s2) * inv * inv * inv * invR + (dvar ? 2.0 * dvar[r] * invR : 0.0); /* :61-63 */
      const double b = -a * m - s1 * inv * invR + (dmean ? dmean[r] * invR : 0.0);                   /* :66-68 */
      for (int64_t i = 0; i < R; ++i) {
        const double g = gamma ? gamma[i] : 1.0;
        dx[(size_t)r * R + i] = (float)(dr[i] * inv * g + a * xr[i] + b); /* :91-92 */
      }
    }
  }
  if (dgamma || dbeta) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < R; ++i) {
      double db = 0, dg = 0;
      for (int64_t r = 0; r < outer; ++r) { /* :106-111 */
        const double inv = 1.0 / sqrt((double)var[r] + eps);
        const double d = dy[(size_t)r * R + i];
        db += d;
        dg += d * ((double)x[(size_t)r * R + i] - mean[r]) * inv;
      }
      if (dbeta) dbeta[i] = (float)db;
      if (dgamma) dgamma[i] = (float)dg;
    }
  }
}

/* ---- GroupNormalization, x[N][C][S], per-channel gamma/beta -------------- */

/* kernel/group_normalization.cuh:32-73 */
NR_EXPORT void nr_gn_forward(const float *x, const float *beta, const float *gamma, float *y,
                             float *mean, float *var, int64_t N, int64_t C, int64_t S,
                             int64_t G, float eps) {
  const int64_t cpg = C / G, R = cpg * S;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < N * G; ++r) {
    const float *xr = x + (size_t)r * R;
    float *yr = y + (size_t)r * R;
    double m, v;
    row_stats(xr, R, &m, &v);
    mean[r] = (float)m;
    var[r] = (float)v;
    const double inv = 1.0 / sqrt(v + eps);
    const int64_t g0 = (r % G) * cpg;
    for (int64_t c = 0; c < cpg; ++c) {
      const double scale = gamma ? gamma[g0 + c] : 1.0;
      const double bias = beta ? beta[g0 + c] : 0.0;
      const double a = scale * inv;    /* :49 */
      const double b = bias - m * a;   /* :50 */
      for (int64_t i = 0; i < S; ++i) yr[c * S + i] = (float)(a * xr[c * S + i] + b); /* :69 */
    }
  }
}

/* kernel/group_normalization.cuh:75-206, reduce_ops/group_normalization.cuh:40-68.
 * scratch: 2*N*C doubles (sum_dy, sum_dyx). */
NR_EXPORT void nr_gn_backward(const float *x, const float *dy, const float *gamma,
                              const float *mean, const float *var, const float *dmean,
                              const float *dvar, float *dx, float *dgamma, float *dbeta,
                              double *scratch, int64_t N, int64_t C, int64_t S, int64_t G,
                              float eps) {
  const int64_t cpg = C / G, R = cpg * S;
  const double invR = 1.0 / (double)R;
  double *sum_dy = scratch, *sum_dyx = scratch + N * C;
#pragma omp parallel for schedule(static)
  for (int64_t p = 0; p < N * C; ++p) {
    double a = 0, b = 0;
    for (int64_t i = 0; i < S; ++i) {
      const double d = dy[(size_t)p * S + i];
      a += d;
      b += d * (double)x[(size_t)p * S + i];
    }
    sum_dy[p] = a;
    sum_dyx[p] = b;
  }
  if (dx) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < N * G; ++r) {
      const double m = mean[r];
      const double inv = 1.0 / sqrt((double)var[r] + eps);
      const int64_t g0 = (r % G) * cpg;
      double s1 = 0, s2 = 0;
      for (int64_t c = 0; c < cpg; ++c) { /* :117-123 */
        const double scale = gamma ? gamma[g0 + c] : 1.0;
        s1 += sum_dy[r * cpg + c] * scale;
        s2 += sum_dyx[r * cpg + c] * scale;
      }
      const double f1 = (s1 * m - s2) * inv * inv * inv * invR + (dvar ? 2.0 * dvar[r] * invR : 0.0); /* :137-140 */
      const double f2 = -f1 * m - s1 * inv * invR + (dmean ? dmean[r] * invR : 0.0);                  /* :142-144 */
      for (int64_t c = 0; c < cpg; ++c) {
        const double gi = (gamma ? gamma[g0 + c] : 1.0) * inv; /* gamma_invstd, :93 */
        const size_t base = (size_t)r * R + c * S;
        for (int64_t i = 0; i < S; ++i) dx[base + i] = (float)(gi * dy[base + i] + f1 * x[base + i] + f2); /* :169-171 */
      }
    }
  }
  if (dgamma || dbeta) {
    for (int64_t c = 0; c < C; ++c) { /* :186-205 */
      double db = 0, dg = 0;
      for (int64_t n = 0; n < N; ++n) {
        const int64_t r = n * G + c / cpg;
        db += sum_dy[n * C + c];
        dg += (sum_dyx[n * C + c] - sum_dy[n * C + c] * mean[r]) / sqrt((double)var[r] + eps);
      }
      if (dbeta) dbeta[c] = (float)db;
      if (dgamma) dgamma[c] = (float)dg;
    }
  }
}

/* ---- InstanceNormalization, x[N][C][S] ---------------------------------- */

/* kernel/instance_normalization.cuh:24-48; bc_*: parameter index row % C, else row */
NR_EXPORT void nr_in_forward(const float *x, const float *beta, const float *gamma, float *y,
                             float *mean, float *var, int64_t N, int64_t C, int64_t S,
                             int bc_gamma, int bc_beta, float eps) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < N * C; ++r) {
    const float *xr = x + (size_t)r * S;
    double m, v;
    row_stats(xr, S, &m, &v);
    mean[r] = (float)m;
    var[r] = (float)v;
    const double inv = 1.0 / sqrt(v + eps);
    const double scale = gamma ? gamma[bc_gamma ? r % C : r] : 1.0;
    const double bias = beta ? beta[bc_beta ? r % C : r] : 0.0;
    for (int64_t i = 0; i < S; ++i) y[(size_t)r * S + i] = (float)(scale * inv * ((double)xr[i] - m) + bias);
  }
}

/* kernel/instance_normalization.cuh:50-121 and the batch sum of
 * generic/instance_normalization.cu:427-464.  dgamma/dbeta have C elements when
 * broadcast, N*C otherwise. */
NR_EXPORT void nr_in_backward(const float *x, const float *dy, const float *gamma,
                              const float *mean, const float *var, const float *dmean,
                              const float *dvar, float *dx, float *dgamma, float *dbeta,
                              double *scratch, int64_t N, int64_t C, int64_t S, int bc_gamma,
                              int bc_beta, float eps) {
  const double invR = 1.0 / (double)S;
  double *row_db = scratch, *row_dg = scratch + N * C;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < N * C; ++r) {
    const double m = mean[r];
    const double inv = 1.0 / sqrt((double)var[r] + eps);
    const double scale = gamma ? gamma[bc_gamma ? r % C : r] : 1.0;
    double sdy = 0, sdyx = 0;
    for (int64_t i = 0; i < S; ++i) {
      const double d = dy[(size_t)r * S + i];
      sdy += d;
      sdyx += d * (double)x[(size_t)r * S + i];
    }
    row_db[r] = sdy;                              /* :110 */
    row_dg[r] = sdyx * inv - sdy * m * inv;       /* :111-112 */
    if (dx) {
      const double a = (sdy * scale * m - sdyx * scale) * inv * inv * inv * invR + (dvar ? 2.0 * dvar[r] * invR : 0.0); /* :63-65 */
      const double b = -a * m - sdy * scale * inv * invR + (dmean ? dmean[r] * invR : 0.0);                           /* :68-70 */
      for (int64_t i = 0; i < S; ++i)
        dx[(size_t)r * S + i] = (float)(dy[(size_t)r * S + i] * inv * scale + a * x[(size_t)r * S + i] + b); /* :94-96 */
    }
  }
  if (dbeta) {
    if (bc_beta) {
      for (int64_t c = 0; c < C; ++c) { double s = 0; for (int64_t n = 0; n < N; ++n) s += row_db[n * C + c]; dbeta[c] = (float)s; }
    } else {
      for (int64_t r = 0; r < N * C; ++r) dbeta[r] = (float)row_db[r];
    }
  }
  if (dgamma) {
    if (bc_gamma) {
      for (int64_t c = 0; c < C; ++c) { double s = 0; for (int64_t n = 0; n < N; ++n) s += row_dg[n * C + c]; dgamma[c] = (float)s; }
    } else {
      for (int64_t r = 0; r < N * C; ++r) dgamma[r] = (float)row_dg[r];
    }
  }
}
