/*
 * oracle.c — CPU restatement of the arithmetic of Hetu's row-wise operator
 * kernels.  TEST INFRASTRUCTURE ONLY: it is the checker the GPU kernels are
 * compared with (tests/, the smoke check, the bench's cpu_baseline leg).  No
 * product code path may call it.
 *
 * Two families:
 *   oracle_*   evaluate the function the reference kernels compute (formula and
 *              semantics of the cited lines) in double precision on inputs that
 *              were already rounded to the storage type; results are returned
 *              unrounded (double) so the caller chooses the comparison.
 *   refcpu_*   fp32 ports of the reference's CPU kernels with the same pass
 *              structure; they are what the bench times as "cpu_baseline".
 *
 * Pinning (see tests/test_oracle.py): closed forms and invariants, brute
 * force on tiny inputs, finite differences for every backward, and
 * cross-checks against an independent library (torch CPU, float64).  The
 * reference repository holds no tests, golden vectors or fixtures for these
 * kernels and cannot be built in this environment, so no function here is
 * pinned by reference-produced data.
 *
 * All citations are relative to the reference tree (hetu/...); "FA!" marks
 * files inside third_party/flash_attn/flash_attn.tar.gz.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------ *
 * bf16 <-> fp32, hetu/core/bfloat16.h:26-53: round to nearest even through
 * the 0x7FFF + lsb bias, NaN -> 0x7FC0.
 * ------------------------------------------------------------------------ */
ORACLE_API uint16_t oracle_f32_to_bf16(float f) {
  if (isnan(f)) return 0x7FC0u;
  uint32_t u;
  memcpy(&u, &f, sizeof(u));
  uint32_t bias = ((u >> 16) & 1u) + 0x7FFFu;
  return (uint16_t)((u + bias) >> 16);
}

ORACLE_API float oracle_bf16_to_f32(uint16_t b) {
  uint32_t u = ((uint32_t)b) << 16;
  float f;
  memcpy(&f, &u, sizeof(f));
  return f;
}

ORACLE_API void oracle_f32_to_bf16_array(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_f32_to_bf16(in[i]);
}

ORACLE_API void oracle_bf16_to_f32_array(const uint16_t* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_bf16_to_f32(in[i]);
}

/* ------------------------------------------------------------------------ *
 * LayerNorm forward.
 *   mean = sum(x)/cols, var = biased variance (>= 0), rstd = 1/sqrt(var+eps),
 *   y = (x - mean) * rstd * gamma + beta
 * hetu/impl/kernel/LayerNorm.cu:15-64 (mean, var = E[x^2]-mean^2 clamped at 0);
 * hetu/impl/kernel/FusedLayerNorm.cu:396-454 (mean, invvar = rsqrt(sigma2+eps)).
 * gamma / beta may be NULL (1 / 0).  Any output pointer may be NULL.
 * ------------------------------------------------------------------------ */
ORACLE_API void oracle_layernorm_fwd(const float* x, const float* gamma, const float* beta,
                                     int64_t rows, int64_t cols, double eps, double* y,
                                     double* mean, double* var, double* rstd) {
  for (int64_t r = 0; r < rows; ++r) {
    const float* xr = x + r * cols;
    double s = 0.0;
    for (int64_t c = 0; c < cols; ++c) s += (double)xr[c];
    const double mu = s / (double)cols;
    double m2 = 0.0;
    for (int64_t c = 0; c < cols; ++c) {
      const double d = (double)xr[c] - mu;
      m2 += d * d;
    }
    double v = m2 / (double)cols;
    if (v < 0.0) v = 0.0;
    const double rs = 1.0 / sqrt(v + eps);
    if (mean) mean[r] = mu;
    if (var) var[r] = v;
    if (rstd) rstd[r] = rs;
    if (y) {
      for (int64_t c = 0; c < cols; ++c) {
        const double g = gamma ? (double)gamma[c] : 1.0;
        const double b = beta ? (double)beta[c] : 0.0;
        y[r * cols + c] = ((double)xr[c] - mu) * rs * g + b;
      }
    }
  }
}

/* clamp_by_magnitude, FusedLayerNorm.cu:486-503 */
static double clamp_by_magnitude(double g, double eps) {
  if (g >= 0.0) return g < eps ? eps : g;
  return g > -eps ? -eps : g;
}

/* ------------------------------------------------------------------------ *
 * LayerNorm backward from saved statistics.
 *   xhat = (x - mean) * rstd
 *   dgamma = sum_rows dy * xhat,  dbeta = sum_rows dy
 *   s1 = sum_cols dy*gamma, s2 = sum_cols dy*gamma*xhat
 *   dx = rstd/cols * (cols*dy*kgamma - s1 - xhat*s2)
 * with kgamma = clamp_gamma ? clamp_by_magnitude(gamma, eps) : gamma.
 * hetu/impl/kernel/LayerNorm.cu:123-233 (the same expression written with
 * ds_/db_, :198-201, no clamp) and FusedLayerNorm.cu:761-965 (clamp applied to
 * the per-element gamma only, :911-938).
 * ------------------------------------------------------------------------ */
ORACLE_API void oracle_layernorm_bwd(const float* dy, const float* x, const float* gamma,
                                     const double* mean, const double* rstd, int64_t rows,
                                     int64_t cols, double eps, int clamp_gamma, double* dx,
                                     double* dgamma, double* dbeta) {
  if (dgamma) memset(dgamma, 0, sizeof(double) * (size_t)cols);
  if (dbeta) memset(dbeta, 0, sizeof(double) * (size_t)cols);
  for (int64_t r = 0; r < rows; ++r) {
    const float* xr = x + r * cols;
    const float* dyr = dy + r * cols;
    const double mu = mean ? mean[r] : 0.0, rs = rstd[r];
    double s1 = 0.0, s2 = 0.0;
    for (int64_t c = 0; c < cols; ++c) {
      const double g = gamma ? (double)gamma[c] : 1.0;
      const double xhat = ((double)xr[c] - mu) * rs;
      s1 += (double)dyr[c] * g;
      s2 += (double)dyr[c] * g * xhat;
      if (dgamma) dgamma[c] += (double)dyr[c] * xhat;
      if (dbeta) dbeta[c] += (double)dyr[c];
    }
    if (dx) {
      for (int64_t c = 0; c < cols; ++c) {
        const double g = gamma ? (double)gamma[c] : 1.0;
        const double kg = clamp_gamma ? clamp_by_magnitude(g, eps) : g;
        const double xhat = ((double)xr[c] - mu) * rs;
        dx[r * cols + c] = rs / (double)cols * ((double)cols * (double)dyr[c] * kg - s1 - xhat * s2);
      }
    }
  }
}

/* Memory-efficient LayerNorm backward: the forward OUTPUT y is given instead
 * of x; xhat = (y - beta) / clamp_by_magnitude(gamma, eps), s2 = sum dy*(y-beta).
 * FusedLayerNorm.cu:538-547 (partials), :790-800, :923-925 (MemoryEfficient). */
ORACLE_API void oracle_layernorm_bwd_memeff(const float* dy, const float* y, const float* gamma,
                                            const float* beta, const double* rstd, int64_t rows,
                                            int64_t cols, double eps, double* dx, double* dgamma,
                                            double* dbeta) {
  if (dgamma) memset(dgamma, 0, sizeof(double) * (size_t)cols);
  if (dbeta) memset(dbeta, 0, sizeof(double) * (size_t)cols);
  for (int64_t r = 0; r < rows; ++r) {
    const float* yr = y + r * cols;
    const float* dyr = dy + r * cols;
    const double rs = rstd[r];
    double s1 = 0.0, s2 = 0.0;
    for (int64_t c = 0; c < cols; ++c) {
      const double g = gamma ? (double)gamma[c] : 1.0;
      const double b = beta ? (double)beta[c] : 0.0;
      const double yb = (double)yr[c] - b;
      s1 += (double)dyr[c] * g;
      s2 += (double)dyr[c] * yb;
      if (dgamma) dgamma[c] += (double)dyr[c] * yb / clamp_by_magnitude(g, eps);
      if (dbeta) dbeta[c] += (double)dyr[c];
    }
    if (dx) {
      for (int64_t c = 0; c < cols; ++c) {
        const double g = gamma ? (double)gamma[c] : 1.0;
        const double b = beta ? (double)beta[c] : 0.0;
        const double kg = clamp_by_magnitude(g, eps);
        const double xhat = ((double)yr[c] - b) / kg;
        dx[r * cols + c] = rs / (double)cols * ((double)cols * (double)dyr[c] * kg - s1 - xhat * s2);
      }
    }
  }
}

/* ------------------------------------------------------------------------ *
 * Dropout-add-LayerNorm / RMSNorm forward (dropout_p = 0, optional residual).
 *   x = x0 + residual; mu = mean(x); m2 = sum (x-mu)^2
 *   rs = 1/sqrt(m2/cols + eps + (is_rms ? mu^2 : 0))
 *   z = gamma * (rs * (x - (is_rms ? 0 : mu))) + beta
 * FA!include/layer_norm/ln_fwd_kernels.cuh:102-177.
 * ------------------------------------------------------------------------ */
ORACLE_API void oracle_dropout_add_ln_fwd(const float* x0, const float* residual,
                                          const float* gamma, const float* beta, int64_t rows,
                                          int64_t cols, double eps, int is_rms, double* z,
                                          double* x_out, double* mu_out, double* rs_out) {
  double* xs = (double*)malloc(sizeof(double) * (size_t)cols);
  for (int64_t r = 0; r < rows; ++r) {
    double s = 0.0;
    for (int64_t c = 0; c < cols; ++c) {
      xs[c] = (double)x0[r * cols + c] + (residual ? (double)residual[r * cols + c] : 0.0);
      if (x_out) x_out[r * cols + c] = xs[c];
      s += xs[c];
    }
    const double mu = s / (double)cols;
    double m2 = 0.0;
    for (int64_t c = 0; c < cols; ++c) m2 += (xs[c] - mu) * (xs[c] - mu);
    const double rs = 1.0 / sqrt(m2 / (double)cols + eps + (is_rms ? mu * mu : 0.0));
    if (mu_out) mu_out[r] = mu;
    if (rs_out) rs_out[r] = rs;
    if (z) {
      for (int64_t c = 0; c < cols; ++c) {
        const double yv = rs * (xs[c] - (is_rms ? 0.0 : mu));
        z[r * cols + c] = (double)gamma[c] * yv + (beta ? (double)beta[c] : 0.0);
      }
    }
  }
  free(xs);
}

/* Dropout-add-LayerNorm / RMSNorm backward (dropout_p = 0).
 *   y = rs*(x - (is_rms?0:mu)); dy = gamma*dz; mdy = mean(dy); mdyy = mean(dy*y)
 *   dx = rs*(dy - (mdyy*y + (is_rms?0:mdy))) (+ dx_in);  dgamma = sum dz*y; dbeta = sum dz
 * FA!include/layer_norm/ln_bwd_kernels.cuh:126-221. */
ORACLE_API void oracle_dropout_add_ln_bwd(const float* dz, const float* dx_in, const float* x,
                                          const double* mu, const double* rs, const float* gamma,
                                          int64_t rows, int64_t cols, int is_rms, double* dx,
                                          double* dgamma, double* dbeta) {
  if (dgamma) memset(dgamma, 0, sizeof(double) * (size_t)cols);
  if (dbeta) memset(dbeta, 0, sizeof(double) * (size_t)cols);
  for (int64_t r = 0; r < rows; ++r) {
    const double m = is_rms ? 0.0 : mu[r], s = rs[r];
    double mdy = 0.0, mdyy = 0.0;
    for (int64_t c = 0; c < cols; ++c) {
      const double y = s * ((double)x[r * cols + c] - m);
      const double dy = (double)gamma[c] * (double)dz[r * cols + c];
      mdy += dy;
      mdyy += dy * y;
      if (dgamma) dgamma[c] += (double)dz[r * cols + c] * y;
      if (dbeta) dbeta[c] += (double)dz[r * cols + c];
    }
    mdy /= (double)cols;
    mdyy /= (double)cols;
    if (dx) {
      for (int64_t c = 0; c < cols; ++c) {
        const double y = s * ((double)x[r * cols + c] - m);
        const double dy = (double)gamma[c] * (double)dz[r * cols + c];
        double v = s * (dy - (mdyy * y + (is_rms ? 0.0 : mdy)));
        if (dx_in) v += (double)dx_in[r * cols + c];
        dx[r * cols + c] = v;
      }
    }
  }
}

/* ------------------------------------------------------------------------ *
 * Softmax along the middle extent of [outer, dim, inner]:
 *   y = exp(x - max) / sum exp(x - max)
 * hetu/impl/kernel/Softmax.cu:148-248.
 * Backward: dx = dy*y - y*sum(dy*y), Softmax.cu:312-362.
 * ------------------------------------------------------------------------ */
ORACLE_API void oracle_softmax_fwd(const float* x, int64_t outer, int64_t dim, int64_t inner,
                                   double* y) {
  for (int64_t o = 0; o < outer; ++o) {
    for (int64_t i = 0; i < inner; ++i) {
      const int64_t base = o * dim * inner + i;
      double m = -INFINITY;
      for (int64_t k = 0; k < dim; ++k) m = fmax(m, (double)x[base + k * inner]);
      double s = 0.0;
      for (int64_t k = 0; k < dim; ++k) s += exp((double)x[base + k * inner] - m);
      for (int64_t k = 0; k < dim; ++k) y[base + k * inner] = exp((double)x[base + k * inner] - m) / s;
    }
  }
}

ORACLE_API void oracle_softmax_bwd(const float* y, const float* dy, int64_t outer, int64_t dim,
                                   int64_t inner, double* dx) {
  for (int64_t o = 0; o < outer; ++o) {
    for (int64_t i = 0; i < inner; ++i) {
      const int64_t base = o * dim * inner + i;
      double dot = 0.0;
      for (int64_t k = 0; k < dim; ++k) dot += (double)y[base + k * inner] * (double)dy[base + k * inner];
      for (int64_t k = 0; k < dim; ++k) {
        const double yv = (double)y[base + k * inner];
        dx[base + k * inner] = (double)dy[base + k * inner] * yv - yv * dot;
      }
    }
  }
}

/* ------------------------------------------------------------------------ *
 * Softmax cross-entropy with sparse int64 labels.
 *   loss[r] = label == ignored ? 0 : log(sum exp(x - max)) + max - x[label]
 * hetu/impl/kernel/SoftmaxCrossEntropySparse.cu:11-55, .cc:11-38.
 * Backward: dx = (softmax - onehot(label)) * grad_loss[r]; zero row when the
 * label is ignored (.cu:93-140, .cc:41-75).
 * ------------------------------------------------------------------------ */
ORACLE_API void oracle_sce_sparse_fwd(const float* x, const int64_t* labels, int64_t rows,
                                      int64_t cols, int64_t ignored, double* loss) {
  for (int64_t r = 0; r < rows; ++r) {
    if (labels[r] == ignored) { loss[r] = 0.0; continue; }
    const float* xr = x + r * cols;
    double m = (double)xr[0];
    for (int64_t c = 1; c < cols; ++c) m = fmax(m, (double)xr[c]);
    double s = 0.0;
    for (int64_t c = 0; c < cols; ++c) s += exp((double)xr[c] - m);
    loss[r] = -(double)xr[labels[r]] + m + log(s);
  }
}

ORACLE_API void oracle_sce_sparse_bwd(const float* x, const int64_t* labels, const float* grad_loss,
                                      int64_t rows, int64_t cols, int64_t ignored, double* dx) {
  for (int64_t r = 0; r < rows; ++r) {
    double* dr = dx + r * cols;
    if (labels[r] == ignored) {
      for (int64_t c = 0; c < cols; ++c) dr[c] = 0.0;
      continue;
    }
    const float* xr = x + r * cols;
    double m = (double)xr[0];
    for (int64_t c = 1; c < cols; ++c) m = fmax(m, (double)xr[c]);
    double s = 0.0;
    for (int64_t c = 0; c < cols; ++c) s += exp((double)xr[c] - m);
    const double g = (double)grad_loss[r];
    for (int64_t c = 0; c < cols; ++c) {
      const double p = exp((double)xr[c] - m) / s;
      dr[c] = (c == labels[r] ? p - 1.0 : p) * g;
    }
  }
}

/* Dense labels: loss = -sum label * log_softmax(x); dx = (softmax - label)*g.
 * hetu/impl/kernel/SoftmaxCrossEntropy.cu:13-73, 91-171 (.cc:12-45, 90-125). */
ORACLE_API void oracle_sce_dense_fwd(const float* x, const float* labels, int64_t rows,
                                     int64_t cols, double* loss) {
  for (int64_t r = 0; r < rows; ++r) {
    const float* xr = x + r * cols;
    double m = (double)xr[0];
    for (int64_t c = 1; c < cols; ++c) m = fmax(m, (double)xr[c]);
    double s = 0.0;
    for (int64_t c = 0; c < cols; ++c) s += exp((double)xr[c] - m);
    const double lse = m + log(s);
    double acc = 0.0;
    for (int64_t c = 0; c < cols; ++c) acc -= (double)labels[r * cols + c] * ((double)xr[c] - lse);
    loss[r] = acc;
  }
}

ORACLE_API void oracle_sce_dense_bwd(const float* x, const float* labels, const float* grad_loss,
                                     int64_t rows, int64_t cols, double* dx) {
  for (int64_t r = 0; r < rows; ++r) {
    const float* xr = x + r * cols;
    double m = (double)xr[0];
    for (int64_t c = 1; c < cols; ++c) m = fmax(m, (double)xr[c]);
    double s = 0.0;
    for (int64_t c = 0; c < cols; ++c) s += exp((double)xr[c] - m);
    for (int64_t c = 0; c < cols; ++c)
      dx[r * cols + c] = (exp((double)xr[c] - m) / s - (double)labels[r * cols + c]) * (double)grad_loss[r];
  }
}

/* ------------------------------------------------------------------------ *
 * Reduce sum / mean over a set of axes of a strided array.  Axes are wrapped
 * to [0, ndim) by the caller, sorted and de-duplicated here
 * (hetu/impl/kernel/Reduce.cuh:765-768); the output is dense with the kept
 * dims in their original order (Reduce.cuh:644-705, out_strides).
 * mean_mode 0: sum / n in double.
 * mean_mode 1: float(sum) * (1.0f / n) evaluated in fp32 as the reference does
 *              (hetu/impl/kernel/ReduceMean.cu:9-33).
 * ------------------------------------------------------------------------ */
ORACLE_API int oracle_reduce(const double* in, int ndim, const int64_t* shape,
                             const int64_t* strides, int naxes, const int64_t* axes, int is_mean,
                             int mean_mode, double* out) {
  if (ndim < 0 || ndim > 16) return -1;
  int red[16] = {0};
  for (int i = 0; i < naxes; ++i) {
    if (axes[i] < 0 || axes[i] >= ndim) return -1;
    red[axes[i]] = 1;
  }
  int64_t n_out = 1, n_red = 1;
  for (int d = 0; d < ndim; ++d) {
    if (red[d]) n_red *= shape[d]; else n_out *= shape[d];
  }
  int64_t idx[16];
  for (int64_t o = 0; o < n_out; ++o) {
    /* decode the kept index (dense, original order) */
    int64_t rem = o, base = 0;
    for (int d = ndim - 1; d >= 0; --d) {
      if (red[d]) continue;
      idx[d] = rem % shape[d];
      rem /= shape[d];
      base += idx[d] * strides[d];
    }
    /* is_mean doubles as the reduction selector: 0 sum, 1 mean, 2 max, 3 min, 4 product
     * (hetu::ReductionType order).  Max / min return a NaN once one has been seen and start from
     * -inf / +inf (ReduceMax.cu:10-25, ReduceMin.cu:10-25); the product starts from 1 (ReduceProd.cu:8-24). */
    double s = is_mean == 2 ? -INFINITY : is_mean == 3 ? INFINITY : is_mean == 4 ? 1.0 : 0.0;
    for (int64_t k = 0; k < n_red; ++k) {
      int64_t r = k, off = base;
      for (int d = ndim - 1; d >= 0; --d) {
        if (!red[d]) continue;
        off += (r % shape[d]) * strides[d];
        r /= shape[d];
      }
      const double v = in[off];
      if (is_mean == 2) s = (isnan(s) || s > v) ? s : v;
      else if (is_mean == 3) s = (isnan(s) || s < v) ? s : v;
      else if (is_mean == 4) s *= v;
      else s += v;
    }
    if (is_mean == 1) {
      if (mean_mode == 1) {
        const float factor = 1.0f / (float)(size_t)n_red;
        s = (double)((float)s * factor);
      } else {
        s = s / (double)n_red;
      }
    }
    out[o] = s;
  }
  return 0;
}

/* ======================================================================== *
 * refcpu_* : fp32 ports of the reference CPU kernels (timed as cpu_baseline).
 * ======================================================================== */

/* LayerNormCpu pass structure, hetu/impl/kernel/LayerNorm.cc:89-137:
 * reduction_mean(x) -> mean; (x-mean)^2 written into the output buffer;
 * reduction_mean -> var; normalise pass with sqrt and divide per element. */
ORACLE_API void refcpu_layernorm_fwd_f32(const float* x, const float* gamma, const float* beta,
                                         int64_t rows, int64_t cols, float eps, float* y,
                                         float* mean, float* var) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    float s = 0.f;
    for (int64_t c = 0; c < cols; ++c) s += x[r * cols + c];
    mean[r] = s / (float)cols;
  }
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < rows * cols; ++i) {
    const float t = x[i] - mean[i / cols];
    y[i] = t * t;
  }
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    float s = 0.f;
    for (int64_t c = 0; c < cols; ++c) s += y[r * cols + c];
    var[r] = s / (float)cols;
  }
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < rows * cols; ++i) {
    const int64_t r = i / cols, c = i % cols;
    y[i] = (x[i] - mean[r]) / sqrtf(var[r] + eps) * gamma[c] + beta[c];
  }
}

/* LayerNormGradientCpu pass structure, hetu/impl/kernel/LayerNorm.cc:177-364: reduction_sum(dy) over rows ->
 * dbias; calculate_gscale (:145-157) writes dy * x_hat into a full-size temporary; reduction_sum -> dscale;
 * reduction_sum(dy) over columns -> db; binary_mul dy * x into a second full-size temporary; reduction_sum ->
 * ds; calculate_grad_kernel (:159-174) writes dx.  The reference's CPU kernel leaves gamma out of db / ds / dx
 * (its GPU kernel does not, LayerNorm.cu:198-201); gamma is applied here, as in the GPU formula:
 *   db = sum_c gamma dy,  ds = sum_c gamma dy x,
 *   dx = gamma dy / sd + ((db mean - ds)(x - mean) / (var + eps) - db) / cols / sd,   sd = sqrt(var + eps). */
ORACLE_API void refcpu_layernorm_bwd_f32(const float* dy, const float* x, const float* gamma,
                                         const float* mean, const float* var, int64_t rows,
                                         int64_t cols, float eps, float* dx, float* dgamma,
                                         float* dbeta) {
  float* t1 = (float*)malloc(sizeof(float) * (size_t)(rows * cols));
  float* t2 = (float*)malloc(sizeof(float) * (size_t)(rows * cols));
  float* ds = (float*)malloc(sizeof(float) * (size_t)rows);
  float* db = (float*)malloc(sizeof(float) * (size_t)rows);
  /* dbias: column sums of dy (the reduction walks rows for a block of columns) */
#pragma omp parallel for schedule(static)
  for (int64_t c = 0; c < cols; ++c) {
    float s = 0.f;
    for (int64_t r = 0; r < rows; ++r) s += dy[r * cols + c];
    dbeta[c] = s;
  }
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < rows * cols; ++i) {
    const int64_t r = i / cols;
    t1[i] = dy[i] * ((x[i] - mean[r]) / sqrtf(var[r] + eps));
  }
#pragma omp parallel for schedule(static)
  for (int64_t c = 0; c < cols; ++c) {
    float s = 0.f;
    for (int64_t r = 0; r < rows; ++r) s += t1[r * cols + c];
    dgamma[c] = s;
  }
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < rows * cols; ++i) {
    const float gd = gamma[i % cols] * dy[i];
    t1[i] = gd;
    t2[i] = gd * x[i];
  }
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    float s1 = 0.f, s2 = 0.f;
    for (int64_t c = 0; c < cols; ++c) { s1 += t1[r * cols + c]; s2 += t2[r * cols + c]; }
    db[r] = s1;
    ds[r] = s2;
  }
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < rows * cols; ++i) {
    const int64_t r = i / cols;
    const float sd = sqrtf(var[r] + eps);
    const float tmp = (db[r] * mean[r] - ds[r]) * (x[i] - mean[r]) / (var[r] + eps);
    dx[i] = t1[i] / sd + ((tmp - db[r]) / (float)cols) / sd;
  }
  free(t1); free(t2); free(ds); free(db);
}

/* RMSNorm has no CPU kernel in the reference (HT_DISPATCH_KERNEL_CUDA_ONLY,
 * hetu/graph/ops/RMSNorm.cc:42): this is the oracle formula in fp32. */
ORACLE_API void refcpu_rmsnorm_fwd_f32(const float* x, const float* gamma, int64_t rows,
                                       int64_t cols, float eps, float* z, float* rs_out) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    float ss = 0.f;
    for (int64_t c = 0; c < cols; ++c) ss += x[r * cols + c] * x[r * cols + c];
    const float rs = 1.0f / sqrtf(ss / (float)cols + eps);
    rs_out[r] = rs;
    for (int64_t c = 0; c < cols; ++c) z[r * cols + c] = gamma[c] * (rs * x[r * cols + c]);
  }
}

ORACLE_API void refcpu_rmsnorm_bwd_f32(const float* dz, const float* x, const float* gamma,
                                       const float* rs, int64_t rows, int64_t cols, float* dx,
                                       float* dgamma) {
  memset(dgamma, 0, sizeof(float) * (size_t)cols);
#pragma omp parallel
  {
    float* local = (float*)calloc((size_t)cols, sizeof(float));
#pragma omp for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
      float mdyy = 0.f;
      for (int64_t c = 0; c < cols; ++c) {
        const float y = rs[r] * x[r * cols + c];
        mdyy += gamma[c] * dz[r * cols + c] * y;
        local[c] += dz[r * cols + c] * y;
      }
      mdyy /= (float)cols;
      for (int64_t c = 0; c < cols; ++c) {
        const float y = rs[r] * x[r * cols + c];
        dx[r * cols + c] = rs[r] * (gamma[c] * dz[r * cols + c] - mdyy * y);
      }
    }
#pragma omp critical
    for (int64_t c = 0; c < cols; ++c) dgamma[c] += local[c];
    free(local);
  }
}

/* SoftmaxCpu calls oneDNN softmax_accurate (hetu/impl/kernel/Softmax.cc:31-45):
 * max, exp and sum, scale — three passes over a row. */
ORACLE_API void refcpu_softmax_fwd_f32(const float* x, int64_t rows, int64_t cols, float* y) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const float* xr = x + r * cols;
    float* yr = y + r * cols;
    float m = xr[0];
    for (int64_t c = 1; c < cols; ++c) m = xr[c] > m ? xr[c] : m;
    float s = 0.f;
    for (int64_t c = 0; c < cols; ++c) { yr[c] = expf(xr[c] - m); s += yr[c]; }
    const float inv = 1.0f / s;
    for (int64_t c = 0; c < cols; ++c) yr[c] *= inv;
  }
}

ORACLE_API void refcpu_softmax_bwd_f32(const float* y, const float* dy, int64_t rows, int64_t cols,
                                       float* dx) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    float dot = 0.f;
    for (int64_t c = 0; c < cols; ++c) dot += y[r * cols + c] * dy[r * cols + c];
    for (int64_t c = 0; c < cols; ++c) dx[r * cols + c] = y[r * cols + c] * (dy[r * cols + c] - dot);
  }
}

/* softmax_cross_entropy_sparse_cpu, hetu/impl/kernel/SoftmaxCrossEntropySparse.cc:11-38
 * (an ignored row is skipped with `continue`; the reference's `return` inside
 * the loop body would stop the whole loop). */
ORACLE_API void refcpu_sce_sparse_fwd_f32(const float* x, const int64_t* labels, int64_t rows,
                                          int64_t cols, int64_t ignored, float* loss) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    if (labels[r] == ignored) { loss[r] = 0.f; continue; }
    const float* xr = x + r * cols;
    float m = xr[0];
    for (int64_t c = 1; c < cols; ++c) m = xr[c] > m ? xr[c] : m;
    float s = 0.f;
    for (int64_t c = 0; c < cols; ++c) s += expf(xr[c] - m);
    loss[r] = -(xr[labels[r]] - m) + logf(s);
  }
}

/* softmax_cross_entropy_sparse_gradient_cpu, hetu/impl/kernel/SoftmaxCrossEntropySparse.cc:41-75: an ignored row
 * is written as zeros (:49-55), every other row as (softmax - onehot) * grad_loss[row] after a max pass and a
 * sum-of-exponentials pass. */
ORACLE_API void refcpu_sce_sparse_bwd_f32(const float* x, const int64_t* labels, const float* grad_loss,
                                          int64_t rows, int64_t cols, int64_t ignored, float* dx) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    float* dr = dx + r * cols;
    if (labels[r] == ignored) { memset(dr, 0, sizeof(float) * (size_t)cols); continue; }
    const float* xr = x + r * cols;
    float m = xr[0];
    for (int64_t c = 1; c < cols; ++c) m = xr[c] > m ? xr[c] : m;
    float s = 0.f;
    for (int64_t c = 0; c < cols; ++c) s += expf(xr[c] - m);
    const float g = grad_loss[r];
    for (int64_t c = 0; c < cols; ++c) dr[c] = (expf(xr[c] - m) / s - (c == labels[r] ? 1.f : 0.f)) * g;
  }
}

/* ReduceCpu -> oneDNN reduction_sum / reduction_mean (hetu/impl/kernel/Reduce.cc:41-68). */
ORACLE_API void refcpu_reduce_sum_axis1_f32(const float* x, int64_t rows, int64_t cols, float* out) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    float s = 0.f;
    for (int64_t c = 0; c < cols; ++c) s += x[r * cols + c];
    out[r] = s;
  }
}

ORACLE_API void refcpu_reduce_sum_axis0_f32(const float* x, int64_t rows, int64_t cols, float* out) {
  memset(out, 0, sizeof(float) * (size_t)cols);
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c) out[c] += x[r * cols + c];
}

ORACLE_API void refcpu_reduce_mean_axis1_f32(const float* x, int64_t rows, int64_t cols, float* out) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    float s = 0.f;
    for (int64_t c = 0; c < cols; ++c) s += x[r * cols + c];
    out[r] = s / (float)cols;
  }
}

ORACLE_API void refcpu_reduce_mean_axis0_f32(const float* x, int64_t rows, int64_t cols, float* out) {
  memset(out, 0, sizeof(float) * (size_t)cols);
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c) out[c] += x[r * cols + c];
  for (int64_t c = 0; c < cols; ++c) out[c] /= (float)rows;
}

ORACLE_API int refcpu_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

ORACLE_API void refcpu_set_num_threads(int n) {
#ifdef _OPENMP
  omp_set_num_threads(n);
#else
  (void)n;
#endif
}
