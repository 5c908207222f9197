/*
 * CPU oracle for anode's GPU operator library (routines_gpu).
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is a plain-C restatement of the
 * arithmetic of the reference's CUDA kernels, used only as the checker in
 * tests, in the smoke check and as the timed CPU baseline of the benchmark.
 * Nothing in the shipped library links, loads or calls it.
 *
 * Two flavours per operator:
 *   *_f32ref : same per-element formula and operation order as the reference
 *              kernel, in fp32.  Reductions follow the reference's order:
 *              tiles of `bs` consecutive fused indices, a stride-halving tree
 *              inside a tile, tiles added sequentially
 *              (routines_gpu/common_reduce.cuh:22-31, batch_norm.cu:37-52).
 *              Where the reference's compiler (nvcc, default -fmad=true,
 *              build.rs:36-47) would contract a multiply feeding an add, an
 *              explicit fmaf() is used; the file is compiled with
 *              -ffp-contract=off so nothing else is fused.
 *   *_f64    : inputs promoted to double, exact formula, plain sums.  This is
 *              the "fp64 host check" for the tolerance class.
 *
 * Index order is first-index-fastest (routines_gpu/common.cuh:87-106):
 *   idx = i0 + dim0 * (i1 + dim1 * i2),  i1 = channel.
 *
 * Pinning status (what fixes each function besides this text):
 *   dequantize, softmax (zeros), softmax_cat_nll (NaN on bad label): the
 *     reference's own known-answer tests, tests/test_gpu.rs:595-758.
 *   upcast, one_hot, label-gather index, arg_max, compare/multiply maps:
 *     exhaustive / brute-force checks on small inputs.
 *   batch-norm pieces, softmax, NLL, F1: closed forms, invariants and
 *     cross-checks against torch in float64 (torch is this build's own
 *     dependency, not the reference's).
 *   quantize_u8, bcast_flat_mult_add, batch_mean_var, online_average and the
 *     other symbols marked ADDITIVE below have no kernel in the reference:
 *     "parity unpinned" by the reference; they are pinned by closed form only
 *     (online_average additionally by tests/test_gpu.rs:561-593).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

ORACLE_API int oracle_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

ORACLE_API void oracle_set_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}

/* ------------------------------------------------------------------------ */
/* the reference's block tree reduction, restated for one tile              */
/* common_reduce.cuh:22-31: for s = bs/2 .. 1: if (t < s && s+t < bs)       */
/*   cache[t] = cache[t] (+|max) cache[t+s]                                 */
/* ------------------------------------------------------------------------ */

static float tile_tree_add(float *cache, uint32_t bs) {
  for (uint32_t s = bs >> 1; s > 0; s >>= 1) {
    for (uint32_t t = 0; t < s; ++t) {
      if (s + t < bs) cache[t] += cache[t + s];
    }
  }
  return cache[0];
}

static float tile_tree_max(float *cache, uint32_t bs) {
  for (uint32_t s = bs >> 1; s > 0; s >>= 1) {
    for (uint32_t t = 0; t < s; ++t) {
      if (s + t < bs) cache[t] = fmaxf(cache[t], cache[t + s]);
    }
  }
  return cache[0];
}

static inline size_t pack3(uint32_t i0, uint32_t d0, uint32_t i1, uint32_t d1, uint32_t i2) {
  return (size_t)i0 + (size_t)d0 * ((size_t)i1 + (size_t)d1 * (size_t)i2);
}

/* Generic per-channel tiled reduction in the reference's order.  TERM is an
 * expression in `idx` (flat element index) giving the fp32 term. */
#define CHANNEL_TILE_REDUCE(d0, d1, d2, bs, PRE, TERM, POST)                      \
  do {                                                                            \
    const uint32_t fused_ = (d0) * (d2);                                          \
    _Pragma("omp parallel")                                                       \
    {                                                                             \
      float *cache = (float *)malloc(sizeof(float) * (bs));                       \
      _Pragma("omp for schedule(static)")                                         \
      for (int64_t c_ = 0; c_ < (int64_t)(d1); ++c_) {                            \
        const uint32_t c = (uint32_t)c_;                                          \
        float accumulator = 0.0f;                                                 \
        PRE;                                                                      \
        for (uint32_t base_ = 0; base_ < fused_; base_ += (bs)) {                 \
          for (uint32_t t_ = 0; t_ < (bs); ++t_) {                                \
            const uint32_t i_ = base_ + t_;                                       \
            if (i_ < fused_) {                                                    \
              const size_t idx = pack3(i_ % (d0), (d0), c, (d1), i_ / (d0));      \
              cache[t_] = (TERM);                                                 \
            } else {                                                              \
              cache[t_] = 0.0f;                                                   \
            }                                                                     \
          }                                                                       \
          accumulator += tile_tree_add(cache, (bs));                              \
        }                                                                         \
        POST;                                                                     \
      }                                                                           \
      free(cache);                                                                \
    }                                                                             \
  } while (0)

/* Plain fp64 per-channel reduction.  TERM is a double expression in `idx`. */
#define CHANNEL_SUM_F64(d0, d1, d2, PRE, TERM, POST)                              \
  do {                                                                            \
    _Pragma("omp parallel for schedule(static)")                                  \
    for (int64_t c_ = 0; c_ < (int64_t)(d1); ++c_) {                              \
      const uint32_t c = (uint32_t)c_;                                            \
      double accumulator = 0.0;                                                   \
      PRE;                                                                        \
      for (uint32_t i2 = 0; i2 < (d2); ++i2) {                                    \
        double inner = 0.0;                                                       \
        for (uint32_t i0 = 0; i0 < (d0); ++i0) {                                  \
          const size_t idx = pack3(i0, (d0), c, (d1), i2);                        \
          inner += (TERM);                                                        \
        }                                                                         \
        accumulator += inner;                                                     \
      }                                                                           \
      POST;                                                                       \
    }                                                                             \
  } while (0)

/* Per-element map over [d0][d1][d2] with the channel index available as c. */
#define CHANNEL_MAP(d0, d1, d2, BODY)                                             \
  do {                                                                            \
    _Pragma("omp parallel for schedule(static) collapse(2)")                      \
    for (int64_t i2_ = 0; i2_ < (int64_t)(d2); ++i2_) {                           \
      for (int64_t c_ = 0; c_ < (int64_t)(d1); ++c_) {                            \
        const uint32_t c = (uint32_t)c_;                                          \
        const size_t row_ = ((size_t)c + (size_t)(d1) * (size_t)i2_) * (size_t)(d0); \
        for (uint32_t i0 = 0; i0 < (d0); ++i0) {                                  \
          const size_t idx = row_ + i0;                                           \
          BODY;                                                                   \
        }                                                                         \
      }                                                                           \
    }                                                                             \
  } while (0)

static inline float norm_of(uint32_t d0, uint32_t d2) {
  /* batch_norm.cu:34: ((float)dim0) * ((float)dim2), an fp32 product */
  return ((float)d0) * ((float)d2);
}

/* The reference calls CUDA's rsqrtf (not reproducible bit-for-bit on other
 * hardware); the restatement uses 1/sqrtf, both correctly rounded. */
static inline float rsqrt_f32(float v) { return 1.0f / sqrtf(v); }

/* ======================================================================== */
/* batch_norm.cu                                                            */
/* ======================================================================== */

/* batch_norm.cu:24-57  mean[c] = (sum x) / (float(dim0)*float(dim2)) */
ORACLE_API void oracle_batch_mean_f32ref(uint32_t d0, uint32_t d1, uint32_t d2, const float *x,
                                         float *mean, uint32_t bs) {
  const float norm1 = norm_of(d0, d2);
  CHANNEL_TILE_REDUCE(d0, d1, d2, bs, (void)0, x[idx], mean[c] = accumulator / norm1);
}

ORACLE_API void oracle_batch_mean_f64(uint32_t d0, uint32_t d1, uint32_t d2, const float *x,
                                      double *mean) {
  const double n = (double)d0 * (double)d2;
  CHANNEL_SUM_F64(d0, d1, d2, (void)0, (double)x[idx], mean[c] = accumulator / n);
}

/* batch_norm.cu:73-95  dx (=|+=) dmean[c] / n */
ORACLE_API void oracle_batch_mean_bwd_f32ref(uint32_t d0, uint32_t d1, uint32_t d2,
                                             const float *dmean, float *dx, int accumulate) {
  const float norm1 = norm_of(d0, d2);
  CHANNEL_MAP(d0, d1, d2, {
    const float v = dmean[c] / norm1;
    dx[idx] = accumulate ? dx[idx] + v : v;
  });
}

ORACLE_API void oracle_batch_mean_bwd_f64(uint32_t d0, uint32_t d1, uint32_t d2, const float *dmean,
                                          const float *dx_in, double *dx, int accumulate) {
  const double n = (double)d0 * (double)d2;
  CHANNEL_MAP(d0, d1, d2, {
    const double v = (double)dmean[c] / n;
    dx[idx] = accumulate ? (double)dx_in[idx] + v : v;
  });
}

/* batch_norm.cu:125-163  var[c] = sum (x-m)^2 / n + eps  (biased, eps inside) */
ORACLE_API void oracle_batch_var_f32ref(uint32_t d0, uint32_t d1, uint32_t d2, float eps,
                                        const float *x, const float *mean, float *var,
                                        uint32_t bs) {
  const float norm2 = norm_of(d0, d2);
  CHANNEL_TILE_REDUCE(d0, d1, d2, bs, const float m = mean[c],
                      (x[idx] - m) * (x[idx] - m), var[c] = accumulator / norm2 + eps);
}

ORACLE_API void oracle_batch_var_f64(uint32_t d0, uint32_t d1, uint32_t d2, float eps,
                                     const float *x, const float *mean, double *var) {
  const double n = (double)d0 * (double)d2;
  CHANNEL_SUM_F64(d0, d1, d2, const double m = (double)mean[c],
                  ((double)x[idx] - m) * ((double)x[idx] - m),
                  var[c] = accumulator / n + (double)eps);
}

/* batch_norm.cu:181-206  dx (=|+=) dvar[c] * (x - m) * 2 / n */
ORACLE_API void oracle_batch_var_bwd_f32ref(uint32_t d0, uint32_t d1, uint32_t d2,
                                            const float *dvar, const float *x, const float *mean,
                                            float *dx, int accumulate) {
  const float norm2 = norm_of(d0, d2);
  CHANNEL_MAP(d0, d1, d2, {
    const float v = dvar[c] * (x[idx] - mean[c]) * 2.0f / norm2;
    dx[idx] = accumulate ? dx[idx] + v : v;
  });
}

ORACLE_API void oracle_batch_var_bwd_f64(uint32_t d0, uint32_t d1, uint32_t d2, const float *dvar,
                                         const float *x, const float *mean, const float *dx_in,
                                         double *dx, int accumulate) {
  const double n = (double)d0 * (double)d2;
  CHANNEL_MAP(d0, d1, d2, {
    const double v = (double)dvar[c] * ((double)x[idx] - (double)mean[c]) * 2.0 / n;
    dx[idx] = accumulate ? (double)dx_in[idx] + v : v;
  });
}

/* batch_norm.cu:240-280  dmean[c] (=|+=) (sum (x - m) * (-dvar[c]*2)) / n */
ORACLE_API void oracle_batch_var_bwd_mean_f32ref(uint32_t d0, uint32_t d1, uint32_t d2,
                                                 const float *dvar, const float *x,
                                                 const float *mean, float *dmean, int accumulate,
                                                 uint32_t bs) {
  const float norm2 = norm_of(d0, d2);
  CHANNEL_TILE_REDUCE(d0, d1, d2, bs, const float m = mean[c];
                      const float dv_term = -dvar[c] * 2.0f, (x[idx] - m) * dv_term, {
                        const float v = accumulator / norm2;
                        dmean[c] = accumulate ? dmean[c] + v : v;
                      });
}

ORACLE_API void oracle_batch_var_bwd_mean_f64(uint32_t d0, uint32_t d1, uint32_t d2,
                                              const float *dvar, const float *x, const float *mean,
                                              const float *dmean_in, double *dmean,
                                              int accumulate) {
  const double n = (double)d0 * (double)d2;
  CHANNEL_SUM_F64(d0, d1, d2, const double m = (double)mean[c];
                  const double dv_term = -(double)dvar[c] * 2.0, ((double)x[idx] - m) * dv_term, {
                    const double v = accumulator / n;
                    dmean[c] = accumulate ? (double)dmean_in[c] + v : v;
                  });
}

/* batch_norm.cu:314-336  y = (x - m) * rsqrtf(var[c]) */
ORACLE_API void oracle_batch_norm_f32ref(uint32_t d0, uint32_t d1, uint32_t d2, const float *x,
                                         const float *mean, const float *var, float *y) {
  CHANNEL_MAP(d0, d1, d2, { y[idx] = (x[idx] - mean[c]) * rsqrt_f32(var[c]); });
}

ORACLE_API void oracle_batch_norm_f64(uint32_t d0, uint32_t d1, uint32_t d2, const float *x,
                                      const float *mean, const float *var, double *y) {
  CHANNEL_MAP(d0, d1, d2,
              { y[idx] = ((double)x[idx] - (double)mean[c]) / sqrt((double)var[c]); });
}

/* batch_norm.cu:354-376  dx (=|+=) dy * rsqrtf(var[c]); the accumulate form is
 * a multiply feeding an add and is restated as one fmaf. */
ORACLE_API void oracle_batch_norm_bwd_f32ref(uint32_t d0, uint32_t d1, uint32_t d2,
                                             const float *dy, const float *var, float *dx,
                                             int accumulate) {
  CHANNEL_MAP(d0, d1, d2, {
    const float rs = rsqrt_f32(var[c]);
    dx[idx] = accumulate ? fmaf(dy[idx], rs, dx[idx]) : dy[idx] * rs;
  });
}

ORACLE_API void oracle_batch_norm_bwd_f64(uint32_t d0, uint32_t d1, uint32_t d2, const float *dy,
                                          const float *var, const float *dx_in, double *dx,
                                          int accumulate) {
  CHANNEL_MAP(d0, d1, d2, {
    const double v = (double)dy[idx] / sqrt((double)var[c]);
    dx[idx] = accumulate ? (double)dx_in[idx] + v : v;
  });
}

/* batch_norm.cu:408-444  dmean[c] (=|+=) sum dy * (-rsqrtf(var[c])) */
ORACLE_API void oracle_batch_norm_bwd_mean_f32ref(uint32_t d0, uint32_t d1, uint32_t d2,
                                                  const float *dy, const float *var, float *dmean,
                                                  int accumulate, uint32_t bs) {
  CHANNEL_TILE_REDUCE(d0, d1, d2, bs, const float v_term = -rsqrt_f32(var[c]), dy[idx] * v_term,
                      dmean[c] = accumulate ? dmean[c] + accumulator : accumulator);
}

ORACLE_API void oracle_batch_norm_bwd_mean_f64(uint32_t d0, uint32_t d1, uint32_t d2,
                                               const float *dy, const float *var,
                                               const float *dmean_in, double *dmean,
                                               int accumulate) {
  CHANNEL_SUM_F64(d0, d1, d2, const double v_term = -1.0 / sqrt((double)var[c]),
                  (double)dy[idx] * v_term,
                  dmean[c] = accumulate ? (double)dmean_in[c] + accumulator : accumulator);
}

/* batch_norm.cu:476-515  dvar[c] (=|+=) sum dy * (x - m) * (-0.5 * rsqrtf(v) / v) */
ORACLE_API void oracle_batch_norm_bwd_var_f32ref(uint32_t d0, uint32_t d1, uint32_t d2,
                                                 const float *dy, const float *x,
                                                 const float *mean, const float *var, float *dvar,
                                                 int accumulate, uint32_t bs) {
  CHANNEL_TILE_REDUCE(d0, d1, d2, bs, const float m = mean[c]; const float v = var[c];
                      const float v_term = -0.5f * rsqrt_f32(v) / v,
                      dy[idx] * (x[idx] - m) * v_term,
                      dvar[c] = accumulate ? dvar[c] + accumulator : accumulator);
}

ORACLE_API void oracle_batch_norm_bwd_var_f64(uint32_t d0, uint32_t d1, uint32_t d2,
                                              const float *dy, const float *x, const float *mean,
                                              const float *var, const float *dvar_in, double *dvar,
                                              int accumulate) {
  CHANNEL_SUM_F64(d0, d1, d2, const double m = (double)mean[c]; const double v = (double)var[c];
                  const double v_term = -0.5 / sqrt(v) / v, (double)dy[idx] * ((double)x[idx] - m) * v_term,
                  dvar[c] = accumulate ? (double)dvar_in[c] + accumulator : accumulator);
}

/* batch_norm.cu:551-587  dvar[c] (=|+=) sum -dy * y * 0.5 / v */
ORACLE_API void oracle_batch_norm_bwd_var_v2_f32ref(uint32_t d0, uint32_t d1, uint32_t d2,
                                                    const float *dy, const float *y,
                                                    const float *var, float *dvar, int accumulate,
                                                    uint32_t bs) {
  CHANNEL_TILE_REDUCE(d0, d1, d2, bs, const float v = var[c], -dy[idx] * y[idx] * 0.5f / v,
                      dvar[c] = accumulate ? dvar[c] + accumulator : accumulator);
}

ORACLE_API void oracle_batch_norm_bwd_var_v2_f64(uint32_t d0, uint32_t d1, uint32_t d2,
                                                 const float *dy, const float *y, const float *var,
                                                 const float *dvar_in, double *dvar,
                                                 int accumulate) {
  CHANNEL_SUM_F64(d0, d1, d2, const double v = (double)var[c],
                  -(double)dy[idx] * (double)y[idx] * 0.5 / v,
                  dvar[c] = accumulate ? (double)dvar_in[c] + accumulator : accumulator);
}

/* ======================================================================== */
/* softmax.cu                                                               */
/* ======================================================================== */

/* softmax.cu:80-130 (and :24-66, which is the single-tile case of the same
 * arithmetic): per row max by tiles, expf(x - max) summed by tiles, z / sum.
 * Element (k, i) lives at k + dim0 * i. */
ORACLE_API void oracle_softmax_f32ref(uint32_t d0, uint32_t d1, const float *x, float *y,
                                      uint32_t bs) {
#pragma omp parallel
  {
    float *cache = (float *)malloc(sizeof(float) * bs);
#pragma omp for schedule(static)
    for (int64_t i_ = 0; i_ < (int64_t)d1; ++i_) {
      const float *xr = x + (size_t)i_ * d0;
      float *yr = y + (size_t)i_ * d0;
      float x_max = -INFINITY;
      for (uint32_t base = 0; base < d0; base += bs) {
        for (uint32_t t = 0; t < bs; ++t) cache[t] = (base + t < d0) ? xr[base + t] : -INFINITY;
        x_max = fmaxf(x_max, tile_tree_max(cache, bs));
      }
      float z_sum = 0.0f;
      for (uint32_t base = 0; base < d0; base += bs) {
        for (uint32_t t = 0; t < bs; ++t)
          cache[t] = (base + t < d0) ? expf(xr[base + t] - x_max) : 0.0f;
        z_sum += tile_tree_add(cache, bs);
      }
      for (uint32_t k = 0; k < d0; ++k) yr[k] = expf(xr[k] - x_max) / z_sum;
    }
    free(cache);
  }
}

ORACLE_API void oracle_softmax_f64(uint32_t d0, uint32_t d1, const float *x, double *y) {
#pragma omp parallel for schedule(static)
  for (int64_t i_ = 0; i_ < (int64_t)d1; ++i_) {
    const float *xr = x + (size_t)i_ * d0;
    double *yr = y + (size_t)i_ * d0;
    double m = -INFINITY;
    for (uint32_t k = 0; k < d0; ++k) m = fmax(m, (double)xr[k]);
    double s = 0.0;
    for (uint32_t k = 0; k < d0; ++k) s += exp((double)xr[k] - m);
    for (uint32_t k = 0; k < d0; ++k) yr[k] = exp((double)xr[k] - m) / s;
  }
}

/* softmax.cu:144-161  nll[i] = label < dim0 ? -logf(p[label + dim0*i]) : NaN */
ORACLE_API void oracle_softmax_cat_nll_f32ref(uint32_t d0, uint32_t d1, const float *softmax,
                                              const uint32_t *cat, float *nll) {
  for (uint32_t i = 0; i < d1; ++i) {
    const uint32_t k = cat[i];
    nll[i] = (k < d0) ? -logf(softmax[(size_t)k + (size_t)d0 * i]) : NAN;
  }
}

ORACLE_API void oracle_softmax_cat_nll_f64(uint32_t d0, uint32_t d1, const float *softmax,
                                           const uint32_t *cat, double *nll) {
  for (uint32_t i = 0; i < d1; ++i) {
    const uint32_t k = cat[i];
    nll[i] = (k < d0) ? -log((double)softmax[(size_t)k + (size_t)d0 * i]) : (double)NAN;
  }
}

/* The flat index of the gathered probability, as an integer (bit-exact class).
 * Returns UINT64_MAX for an out-of-range label. */
ORACLE_API void oracle_softmax_cat_gather_index(uint32_t d0, uint32_t d1, const uint32_t *cat,
                                                uint64_t *index) {
  for (uint32_t i = 0; i < d1; ++i)
    index[i] = (cat[i] < d0) ? (uint64_t)cat[i] + (uint64_t)d0 * i : UINT64_MAX;
}

/* softmax.cu:177-195  dx[k,i] (=|+=) dy[i] * (p[k,i] - float(label[i]==k));
 * the accumulate form is restated as one fmaf. */
ORACLE_API void oracle_softmax_cat_nll_bwd_f32ref(uint32_t d0, uint32_t d1, const float *dy,
                                                  const float *softmax, const uint32_t *cat,
                                                  float *dx, int accumulate) {
#pragma omp parallel for schedule(static)
  for (int64_t i_ = 0; i_ < (int64_t)d1; ++i_) {
    const uint32_t i = (uint32_t)i_;
    for (uint32_t k = 0; k < d0; ++k) {
      const size_t idx = (size_t)k + (size_t)d0 * i;
      const float t = softmax[idx] - (float)(cat[i] == k);
      dx[idx] = accumulate ? fmaf(dy[i], t, dx[idx]) : dy[i] * t;
    }
  }
}

ORACLE_API void oracle_softmax_cat_nll_bwd_f64(uint32_t d0, uint32_t d1, const float *dy,
                                               const float *softmax, const uint32_t *cat,
                                               const float *dx_in, double *dx, int accumulate) {
#pragma omp parallel for schedule(static)
  for (int64_t i_ = 0; i_ < (int64_t)d1; ++i_) {
    const uint32_t i = (uint32_t)i_;
    for (uint32_t k = 0; k < d0; ++k) {
      const size_t idx = (size_t)k + (size_t)d0 * i;
      const double v = (double)dy[i] * ((double)softmax[idx] - (double)(cat[i] == k));
      dx[idx] = accumulate ? (double)dx_in[idx] + v : v;
    }
  }
}

/* softmax.cu:227-262  channel-axis softmax: element (p,k,n) at p + P*(k + C*n),
 * one serial pass per pixel for max, exp-sum and normalise. */
ORACLE_API void oracle_softmax_nd_f32ref(uint32_t P, uint32_t C, uint32_t N, const float *x,
                                         float *y) {
#pragma omp parallel for schedule(static) collapse(2)
  for (int64_t n = 0; n < (int64_t)N; ++n) {
    for (int64_t p = 0; p < (int64_t)P; ++p) {
      const size_t base = (size_t)p + (size_t)P * (size_t)C * (size_t)n;
      float m = -INFINITY;
      for (uint32_t k = 0; k < C; ++k) m = fmaxf(m, x[base + (size_t)P * k]);
      float s = 0.0f;
      for (uint32_t k = 0; k < C; ++k) s += expf(x[base + (size_t)P * k] - m);
      for (uint32_t k = 0; k < C; ++k)
        y[base + (size_t)P * k] = expf(x[base + (size_t)P * k] - m) / s;
    }
  }
}

ORACLE_API void oracle_softmax_nd_f64(uint32_t P, uint32_t C, uint32_t N, const float *x,
                                      double *y) {
#pragma omp parallel for schedule(static) collapse(2)
  for (int64_t n = 0; n < (int64_t)N; ++n) {
    for (int64_t p = 0; p < (int64_t)P; ++p) {
      const size_t base = (size_t)p + (size_t)P * (size_t)C * (size_t)n;
      double m = -INFINITY;
      for (uint32_t k = 0; k < C; ++k) m = fmax(m, (double)x[base + (size_t)P * k]);
      double s = 0.0;
      for (uint32_t k = 0; k < C; ++k) s += exp((double)x[base + (size_t)P * k] - m);
      for (uint32_t k = 0; k < C; ++k)
        y[base + (size_t)P * k] = exp((double)x[base + (size_t)P * k] - m) / s;
    }
  }
}

/* softmax.cu:278-298  nll[p,n] = label < C ? -logf(prob[p + P*(label + C*n)]) : NaN */
ORACLE_API void oracle_softmax_nd_cat_nll_f32ref(uint32_t P, uint32_t C, uint32_t N,
                                                 const float *softmax, const uint32_t *cat,
                                                 float *nll) {
#pragma omp parallel for schedule(static)
  for (int64_t i_ = 0; i_ < (int64_t)P * (int64_t)N; ++i_) {
    const size_t i = (size_t)i_;
    const uint32_t k = cat[i];
    const size_t p = i % P, n = i / P;
    nll[i] = (k < C) ? -logf(softmax[p + (size_t)P * ((size_t)k + (size_t)C * n)]) : NAN;
  }
}

ORACLE_API void oracle_softmax_nd_cat_nll_f64(uint32_t P, uint32_t C, uint32_t N,
                                              const float *softmax, const uint32_t *cat,
                                              double *nll) {
#pragma omp parallel for schedule(static)
  for (int64_t i_ = 0; i_ < (int64_t)P * (int64_t)N; ++i_) {
    const size_t i = (size_t)i_;
    const uint32_t k = cat[i];
    const size_t p = i % P, n = i / P;
    nll[i] = (k < C) ? -log((double)softmax[p + (size_t)P * ((size_t)k + (size_t)C * n)])
                     : (double)NAN;
  }
}

ORACLE_API void oracle_softmax_nd_cat_gather_index(uint32_t P, uint32_t C, uint32_t N,
                                                   const uint32_t *cat, uint64_t *index) {
  for (size_t i = 0; i < (size_t)P * N; ++i) {
    const size_t p = i % P, n = i / P;
    index[i] = (cat[i] < C) ? (uint64_t)(p + (size_t)P * ((size_t)cat[i] + (size_t)C * n))
                            : UINT64_MAX;
  }
}

/* softmax.cu:315-334  dx[p,k,n] (=|+=) dy[p,n] * (prob - float(label[p,n]==k)) */
ORACLE_API void oracle_softmax_nd_cat_nll_bwd_f32ref(uint32_t P, uint32_t C, uint32_t N,
                                                     const float *dy, const float *softmax,
                                                     const uint32_t *cat, float *dx,
                                                     int accumulate) {
#pragma omp parallel for schedule(static) collapse(2)
  for (int64_t n = 0; n < (int64_t)N; ++n) {
    for (int64_t k = 0; k < (int64_t)C; ++k) {
      for (uint32_t p = 0; p < P; ++p) {
        const size_t i = (size_t)p + (size_t)P * (size_t)n;
        const size_t idx = (size_t)p + (size_t)P * ((size_t)k + (size_t)C * (size_t)n);
        const float t = softmax[idx] - (float)(cat[i] == (uint32_t)k);
        dx[idx] = accumulate ? fmaf(dy[i], t, dx[idx]) : dy[i] * t;
      }
    }
  }
}

ORACLE_API void oracle_softmax_nd_cat_nll_bwd_f64(uint32_t P, uint32_t C, uint32_t N,
                                                  const float *dy, const float *softmax,
                                                  const uint32_t *cat, const float *dx_in,
                                                  double *dx, int accumulate) {
#pragma omp parallel for schedule(static) collapse(2)
  for (int64_t n = 0; n < (int64_t)N; ++n) {
    for (int64_t k = 0; k < (int64_t)C; ++k) {
      for (uint32_t p = 0; p < P; ++p) {
        const size_t i = (size_t)p + (size_t)P * (size_t)n;
        const size_t idx = (size_t)p + (size_t)P * ((size_t)k + (size_t)C * (size_t)n);
        const double v = (double)dy[i] * ((double)softmax[idx] - (double)(cat[i] == (uint32_t)k));
        dx[idx] = accumulate ? (double)dx_in[idx] + v : v;
      }
    }
  }
}

/* ======================================================================== */
/* flat_map.cu / flat_join.cu                                               */
/* ======================================================================== */

enum {
  ORACLE_MAP_COPY = 0,
  ORACLE_MAP_MODULUS = 1,
  ORACLE_MAP_SQUARE = 2,
  ORACLE_MAP_SQRT = 3,
  ORACLE_MAP_POSITIVE_CLIP = 4,
  ORACLE_MAP_LOGISTIC = 5,
  ORACLE_MAP_UNIT_STEP = 6,
  ORACLE_MAP_NORMAL_CDF = 7,
  ORACLE_MAP_TANH = 8,
  ORACLE_MAP_RCOSH2 = 9,
  ORACLE_MAP_LEAKY_RELU = 10, /* uses c */
  /* declared in build.rs:101-102 but never given a wrapper in the reference;
   * functor bodies at flat_map.cu:242-278 */
  ORACLE_MAP_LOG_POSITIVE_CLIP = 11,
  ORACLE_MAP_POSITIVE_RECIPROCAL = 12,
};

/* flat_map.cu:44-52, 121-323.  Safe for y == x. */
ORACLE_API int oracle_flat_map_f32ref(int op, uint32_t len, float c, const float *x, float *y) {
  if (op < 0 || op > ORACLE_MAP_POSITIVE_RECIPROCAL) return -1;
#pragma omp parallel for schedule(static)
  for (int64_t i_ = 0; i_ < (int64_t)len; ++i_) {
    const float v = x[i_];
    float r;
    switch (op) {
      case ORACLE_MAP_COPY: r = v; break;
      case ORACLE_MAP_MODULUS: r = fabsf(v); break;
      case ORACLE_MAP_SQUARE: r = v * v; break;
      case ORACLE_MAP_SQRT: r = sqrtf(v); break;
      case ORACLE_MAP_POSITIVE_CLIP: r = v * (float)(v > 0.0f); break;
      case ORACLE_MAP_LOGISTIC: r = 1.0f / (1.0f + expf(-v)); break;
      case ORACLE_MAP_UNIT_STEP: r = (float)(v > 0.0f); break;
      case ORACLE_MAP_NORMAL_CDF: r = 0.5f * (1.0f + erff(v * 0.7071067811865475f)); break;
      case ORACLE_MAP_TANH: r = tanhf(v); break;
      case ORACLE_MAP_RCOSH2: {
        const float ch = coshf(v);
        r = 1.0f / (ch * ch);
        break;
      }
      case ORACLE_MAP_LEAKY_RELU: {
        const float mask = (float)(v > 0.0f);
        r = fmaf(1.0f - mask, c, mask) * v;
        break;
      }
      case ORACLE_MAP_LOG_POSITIVE_CLIP: r = (v > 0.0f) ? logf(v) : -INFINITY; break;
      default: r = (v > 0.0f) ? 1.0f / v : 0.0f; break;
    }
    y[i_] = r;
  }
  return 0;
}

ORACLE_API int oracle_flat_map_f64(int op, uint32_t len, float c, const float *x, double *y) {
  if (op < 0 || op > ORACLE_MAP_POSITIVE_RECIPROCAL) return -1;
#pragma omp parallel for schedule(static)
  for (int64_t i_ = 0; i_ < (int64_t)len; ++i_) {
    const double v = (double)x[i_];
    double r;
    switch (op) {
      case ORACLE_MAP_COPY: r = v; break;
      case ORACLE_MAP_MODULUS: r = fabs(v); break;
      case ORACLE_MAP_SQUARE: r = v * v; break;
      case ORACLE_MAP_SQRT: r = sqrt(v); break;
      case ORACLE_MAP_POSITIVE_CLIP: r = v * (double)(v > 0.0); break;
      case ORACLE_MAP_LOGISTIC: r = 1.0 / (1.0 + exp(-v)); break;
      case ORACLE_MAP_UNIT_STEP: r = (double)(v > 0.0); break;
      case ORACLE_MAP_NORMAL_CDF: r = 0.5 * (1.0 + erf(v * 0.70710678118654752440)); break;
      case ORACLE_MAP_TANH: r = tanh(v); break;
      case ORACLE_MAP_RCOSH2: {
        const double ch = cosh(v);
        r = 1.0 / (ch * ch);
        break;
      }
      case ORACLE_MAP_LEAKY_RELU: r = (v > 0.0) ? v : (double)c * v; break;
      case ORACLE_MAP_LOG_POSITIVE_CLIP: r = (v > 0.0) ? log(v) : -INFINITY; break;
      default: r = (v > 0.0) ? 1.0 / v : 0.0; break;
    }
    y[i_] = r;
  }
  return 0;
}

enum {
  ORACLE_MAPBWD_POSITIVE_CLIP = 0, /* flat_map.cu:187-194 */
  ORACLE_MAPBWD_LOGISTIC = 1,      /* flat_map.cu:217-225 */
  ORACLE_MAPBWD_LEAKY_RELU = 2,    /* flat_map.cu:60-69 */
  ORACLE_JOIN_COPY_UNIT_STEP = 3,  /* flat_join.cu:28-36: a = x1, b = x2 */
};

/* Two-input maps out = f(a, b): backward maps take (a, b) = (dy, y).
 * Safe for out == a (in-place positive_clip backward). */
ORACLE_API int oracle_flat_map2_f32ref(int op, uint32_t len, float c, const float *a,
                                       const float *b, float *out) {
  if (op < 0 || op > ORACLE_JOIN_COPY_UNIT_STEP) return -1;
#pragma omp parallel for schedule(static)
  for (int64_t i_ = 0; i_ < (int64_t)len; ++i_) {
    const float a_i = a[i_], b_i = b[i_];
    float r;
    switch (op) {
      case ORACLE_MAPBWD_POSITIVE_CLIP: r = a_i * (float)(b_i > 0.0f); break;
      case ORACLE_MAPBWD_LOGISTIC: r = a_i * b_i * (1.0f - b_i); break;
      case ORACLE_MAPBWD_LEAKY_RELU: {
        const float mask = (float)(b_i > 0.0f);
        r = fmaf(1.0f - mask, c, mask) * a_i;
        break;
      }
      default: r = a_i * (float)(b_i > 0.0f); break;
    }
    out[i_] = r;
  }
  return 0;
}

/* ======================================================================== */
/* cast.cu, quantize.cu, discrete.cu                                        */
/* ======================================================================== */

/* cast.cu:23-31 */
ORACLE_API void oracle_upcast_u8_u32(uint32_t len, const uint8_t *x, uint32_t *y) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < (int64_t)len; ++i) y[i] = (uint32_t)x[i];
}

/* quantize.cu:23-34  scale = (hi-lo)/255; y = float(x)*scale + lo, one FMA */
ORACLE_API void oracle_dequantize_u8_f32ref(uint32_t len, float lo, float hi, const uint8_t *x,
                                            float *y) {
  const float scale = (hi - lo) / 255.0f;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < (int64_t)len; ++i) y[i] = fmaf((float)x[i], scale, lo);
}

/* The same formula with the multiply and the add rounded separately; used by
 * tests to show on which inputs the contraction choice is visible. */
ORACLE_API void oracle_dequantize_u8_f32_unfused(uint32_t len, float lo, float hi,
                                                 const uint8_t *x, float *y) {
  const float scale = (hi - lo) / 255.0f;
  for (uint32_t i = 0; i < len; ++i) {
    volatile float prod = (float)x[i] * scale;
    y[i] = prod + lo;
  }
}

/* discrete.cu:21-46  y[i0,k,i2] = (label[i0 + dim0*i2] == k) ? 1 : 0 */
ORACLE_API void oracle_discrete_one_hot(uint32_t d0, uint32_t K, uint32_t d2, const uint32_t *cat,
                                        float *y) {
#pragma omp parallel for schedule(static) collapse(2)
  for (int64_t i2 = 0; i2 < (int64_t)d2; ++i2) {
    for (int64_t k = 0; k < (int64_t)K; ++k) {
      for (uint32_t i0 = 0; i0 < d0; ++i0) {
        const size_t src = (size_t)i0 + (size_t)d0 * (size_t)i2;
        y[pack3(i0, d0, (uint32_t)k, K, (uint32_t)i2)] = (cat[src] == (uint32_t)k) ? 1.0f : 0.0f;
      }
    }
  }
}

/* ======================================================================== */
/* f1.cu                                                                    */
/* ======================================================================== */

/* f1.cu:23-71  y[k,n] = -(2*sum x*t + eps) / (sum (x+t) + eps), sums over dim0
 * by tiles; 2*num + eps is a multiply feeding an add (restated as fmaf, which
 * rounds identically because doubling is exact). */
ORACLE_API void oracle_smooth_negative_f1_loss_f32ref(uint32_t d0, uint32_t K, uint32_t d2,
                                                      float eps, const float *x,
                                                      const float *target, float *y,
                                                      uint32_t bs) {
  const uint32_t rows = K * d2;
#pragma omp parallel
  {
    float *nc = (float *)malloc(sizeof(float) * bs);
    float *dc = (float *)malloc(sizeof(float) * bs);
#pragma omp for schedule(static)
    for (int64_t r = 0; r < (int64_t)rows; ++r) {
      const float *xr = x + (size_t)r * d0;
      const float *tr = target + (size_t)r * d0;
      float num = 0.0f, den = 0.0f;
      for (uint32_t base = 0; base < d0; base += bs) {
        for (uint32_t t = 0; t < bs; ++t) {
          if (base + t < d0) {
            nc[t] = xr[base + t] * tr[base + t];
            dc[t] = xr[base + t] + tr[base + t];
          } else {
            nc[t] = 0.0f;
            dc[t] = 0.0f;
          }
        }
        num += tile_tree_add(nc, bs);
        den += tile_tree_add(dc, bs);
      }
      y[r] = -fmaf(2.0f, num, eps) / (den + eps);
    }
    free(nc);
    free(dc);
  }
}

ORACLE_API void oracle_smooth_negative_f1_loss_f64(uint32_t d0, uint32_t K, uint32_t d2, float eps,
                                                   const float *x, const float *target,
                                                   double *y) {
  const uint32_t rows = K * d2;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < (int64_t)rows; ++r) {
    const float *xr = x + (size_t)r * d0;
    const float *tr = target + (size_t)r * d0;
    double num = 0.0, den = 0.0;
    for (uint32_t i = 0; i < d0; ++i) {
      num += (double)xr[i] * (double)tr[i];
      den += (double)xr[i] + (double)tr[i];
    }
    y[r] = -(2.0 * num + (double)eps) / (den + (double)eps);
  }
}

/* f1.cu:89-115  dx = dy[k,n] * -(2 t (t+eps) - eps) / (x+t+eps)^2; the
 * numerator's multiply-subtract is restated as one fmaf. */
ORACLE_API void oracle_smooth_negative_f1_loss_bwd_f32ref(uint32_t d0, uint32_t K, uint32_t d2,
                                                          float eps, const float *dy,
                                                          const float *x, const float *target,
                                                          float *dx) {
  const uint32_t rows = K * d2;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < (int64_t)rows; ++r) {
    for (uint32_t i = 0; i < d0; ++i) {
      const size_t idx = (size_t)r * d0 + i;
      const float tg = target[idx];
      const float numer = fmaf(2.0f * tg, tg + eps, -eps);
      const float denom = x[idx] + tg + eps;
      dx[idx] = dy[r] * -numer / (denom * denom);
    }
  }
}

ORACLE_API void oracle_smooth_negative_f1_loss_bwd_f64(uint32_t d0, uint32_t K, uint32_t d2,
                                                       float eps, const float *dy, const float *x,
                                                       const float *target, double *dx) {
  const uint32_t rows = K * d2;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < (int64_t)rows; ++r) {
    for (uint32_t i = 0; i < d0; ++i) {
      const size_t idx = (size_t)r * d0 + i;
      const double tg = (double)target[idx], e = (double)eps;
      const double numer = 2.0 * tg * (tg + e) - e;
      const double denom = (double)x[idx] + tg + e;
      dx[idx] = (double)dy[r] * -numer / (denom * denom);
    }
  }
}

/* ======================================================================== */
/* host-side argmax, src/utils/mod.rs:31-41                                 */
/* ======================================================================== */

/* first index of the strict maximum; starts from (-inf, 0); NaN never wins */
ORACLE_API uint64_t oracle_arg_max(const float *xs, uint64_t len) {
  float top_x = -INFINITY;
  uint64_t top_k = 0;
  for (uint64_t k = 0; k < len; ++k) {
    if (xs[k] > top_x) {
      top_x = xs[k];
      top_k = k;
    }
  }
  return top_k;
}

/* row-wise form for logits stored as [K classes fastest][rows] */
ORACLE_API void oracle_arg_max_rows(uint32_t d0, uint32_t d1, const float *x, uint32_t *out) {
  for (uint32_t i = 0; i < d1; ++i) out[i] = (uint32_t)oracle_arg_max(x + (size_t)i * d0, d0);
}

/* ======================================================================== */
/* ADDITIVE symbols: no kernel in the reference ("parity unpinned" by it).  */
/* ======================================================================== */

/* inverse of dequantize: q = clamp(rint((x - lo) / scale), 0, 255), rint =
 * round-half-even, NaN -> 0, scale = (hi - lo) / 255 */
ORACLE_API void oracle_quantize_u8(uint32_t len, float lo, float hi, const float *x, uint8_t *y) {
  const float scale = (hi - lo) / 255.0f;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < (int64_t)len; ++i) {
    float q = rintf((x[i] - lo) / scale);
    if (!(q >= 0.0f)) q = 0.0f; /* also catches NaN */
    if (q > 255.0f) q = 255.0f;
    y[i] = (uint8_t)q;
  }
}

/* the commented-out declaration lib.h:223-232: y[i,b,o] = lx[b]*rx[i,b,o] + shift[b]
 * (one fmaf); shift == NULL gives the multiply-only form lib.h:214-222 */
ORACLE_API void oracle_bcast_flat_mult_add(uint32_t inner, uint32_t bcast, uint32_t outer,
                                           const float *lx, const float *rx, const float *shift,
                                           float *y) {
  CHANNEL_MAP(inner, bcast, outer,
              { y[idx] = shift ? fmaf(lx[c], rx[idx], shift[c]) : lx[c] * rx[idx]; });
}

/* fused u8 image normalisation: y = a[c] * float(q) + b[c] (one fmaf) */
ORACLE_API void oracle_bcast_dequantize_u8(uint32_t inner, uint32_t bcast, uint32_t outer,
                                           const float *a, const float *b, const uint8_t *q,
                                           float *y) {
  CHANNEL_MAP(inner, bcast, outer, { y[idx] = fmaf(a[c], (float)q[idx], b[c]); });
}

/* single-pass statistics: mean and biased variance + eps, in double */
ORACLE_API void oracle_batch_mean_var_f64(uint32_t d0, uint32_t d1, uint32_t d2, float eps,
                                          const float *x, double *mean, double *var) {
  oracle_batch_mean_f64(d0, d1, d2, x, mean);
  const double n = (double)d0 * (double)d2;
  CHANNEL_SUM_F64(d0, d1, d2, const double m = mean[c],
                  ((double)x[idx] - m) * ((double)x[idx] - m),
                  var[c] = accumulator / n + (double)eps);
}

/* the commented-out declarations lib.h:408-430: y[b] = sum_{a,c} x[a,b,c] (or of x^2), in double */
ORACLE_API void oracle_channel_sum_f64(uint32_t d0, uint32_t d1, uint32_t d2, int square, const float *x,
                                       double *y) {
  CHANNEL_SUM_F64(d0, d1, d2, (void)0, square ? (double)x[idx] * (double)x[idx] : (double)x[idx],
                  y[c] = accumulator);
}

/* batch_norm followed by the per-channel affine: y = fma((x-m)*rs, gamma[c], beta[c]) */
ORACLE_API void oracle_batch_norm_affine_f32ref(uint32_t d0, uint32_t d1, uint32_t d2, const float *x,
                                                const float *mean, const float *var, const float *gamma,
                                                const float *beta, float *y) {
  CHANNEL_MAP(d0, d1, d2,
              { y[idx] = fmaf((x[idx] - mean[c]) * rsqrt_f32(var[c]), gamma[c], beta[c]); });
}

ORACLE_API void oracle_batch_norm_affine_f64(uint32_t d0, uint32_t d1, uint32_t d2, const float *x,
                                             const float *mean, const float *var, const float *gamma,
                                             const float *beta, double *y) {
  CHANNEL_MAP(d0, d1, d2, {
    y[idx] = ((double)x[idx] - (double)mean[c]) / sqrt((double)var[c]) * (double)gamma[c] + (double)beta[c];
  });
}

/* running statistics, semantics fixed by tests/test_gpu.rs:561-593:
 * y <- y + rate * (x - y) */
ORACLE_API void oracle_online_average(uint32_t len, float rate, const float *x, float *y) {
  for (uint32_t i = 0; i < len; ++i) y[i] = fmaf(rate, x[i] - y[i], y[i]);
}

/* --------------------------------------------------------------------------
 * The neighbours anode takes from gpudevicemem (no source in the reference
 * tree): closed forms implied by the call sites in src/ops_gpu.rs.
 * Parity unpinned by the reference except for the fills and the sum-join
 * value of tests/test_gpu.rs:245-353.
 * -------------------------------------------------------------------------- */

/* src/ops_gpu.rs:7486: y = sum_i x[i], here as the fp64 sum */
ORACLE_API double oracle_sum_packed_f64(uint32_t len, const float *x) {
  double s = 0.0;
  for (uint32_t i = 0; i < len; ++i) s += (double)x[i];
  return s;
}

/* src/ops_gpu.rs:5886: y <- y + rate * x, one fmaf */
ORACLE_API void oracle_online_add(uint32_t len, float rate, const float *x, float *y) {
  for (uint32_t i = 0; i < len; ++i) y[i] = fmaf(rate, x[i], y[i]);
}

/* src/ops_gpu.rs:5972, src/ops.rs:1425-1430: y <- rate * y + x, one fmaf (momentum buffer) */
ORACLE_API void oracle_online_discount(uint32_t len, float rate, const float *x, float *y) {
  for (uint32_t i = 0; i < len; ++i) y[i] = fmaf(rate, y[i], x[i]);
}

/* src/ops_gpu.rs:9592: y[a,b] = x[a,b] / r[b], IEEE division */
ORACLE_API void oracle_flat_bcast_rdiv(uint32_t inner, uint32_t outer, const float *x, const float *r,
                                       float *y) {
  for (uint32_t b = 0; b < outer; ++b)
    for (uint32_t a = 0; a < inner; ++a) y[a + (size_t)inner * b] = x[a + (size_t)inner * b] / r[b];
}
