/*
 * CPU oracle in C for raf.op.sgd and raf.op.lans -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A second, independent restatement of the same rules as sgd_f32.py / lans_f64.py, fast enough
 * to check the GPU at the full benchmark sizes and to serve as the timed CPU baseline.  Only
 * tests, the smoke check and the benchmark's cpu_baseline leg may load the library built from
 * this file.
 *
 * Build: see oracle/Makefile.  -ffp-contract=off is mandatory: the SGD rule is four separately
 * rounded fp32 operations (python/raf/_tvm_op/sgd.py:16-30 lowered for a plain "llvm" target,
 * include/raf/device.h:97-104) and a fused multiply-add would change bit patterns.
 *
 * Reference lines followed (relative to the reference tree):
 *   SGD      python/raf/_tvm_op/sgd.py:13-30
 *   scalars  src/op/dialect/cuda/lans.cc:94-109
 *   norms    src/op/dialect/cuda/kernels/multi_tensor_lans.cu:95-185
 *   stage 1  src/op/dialect/cuda/kernels/multi_tensor_lans.cu:283-307 (:264-269 for wd == 0)
 *   stage 2  src/op/dialect/cuda/kernels/multi_tensor_lans.cu:346-352, :386
 *   order    src/op/dialect/cuda/kernels/multi_tensor_lans.cu:420-447
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ SGD */

/* v1 = fl(fl(mu32*v0) + dx) ; x1 = fl(x0 - fl(lr32*v1)).  mu, lr arrive as the schema's doubles
 * and are rounded once to fp32 like tir.const(..., "float32") does (sgd.py:18-19). */
void oracle_sgd_f32(const float* x0, const float* dx, const float* v0, float* v1, float* x1,
                    int64_t n, double learning_rate, double mu, int threads) {
  const float lr32 = (float)learning_rate;
  const float mu32 = (float)mu;
  (void)threads;
#pragma omp parallel for schedule(static) num_threads(threads > 0 ? threads : 1)
  for (int64_t i = 0; i < n; ++i) {
    float t = mu32 * v0[i]; /* -ffp-contract=off keeps the four roundings apart */
    float vn = t + dx[i];
    float s = lr32 * vn;
    v1[i] = vn;
    x1[i] = x0[i] - s;
  }
}

/* ------------------------------------------------------------------ LANS */

typedef struct {
  float learning_rate, beta1, beta2, eps, weight_decay;
  int32_t bias_correction, grad_averaging, mode, normalize_grad;
  float grad_unscale;
} oracle_lans_hparams;

/* IEEE binary16 -> float, bit-level (no reliance on compiler half support). */
static float half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do {
        man <<= 1;
        ++e;
      } while (!(man & 0x400u));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* bfloat16 -> float: the pattern is the upper half of the fp32 word. */
static float bf16_to_float(uint16_t h) {
  uint32_t bits = (uint32_t)h << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* float -> IEEE binary16, round to nearest even, bit-level.  This is the `cast(new_w, "float16")`
 * of the mixed-precision wrapper (python/raf/optim/lans.py:289-291). */
static uint16_t float_to_half(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  const uint32_t ax = x & 0x7fffffffu;
  if (ax > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);  /* NaN */
  if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 rounds to infinity */
  if (ax <= 0x33000000u) return sign;                       /* <= 2^-25 rounds to zero */
  const uint32_t exp = ax >> 23;
  if (exp < 113) { /* below 2^-14: a binary16 subnormal, unit 2^-24 */
    const uint32_t man = (ax & 0x7fffffu) | 0x800000u;
    const uint32_t shift = 126 - exp; /* 14 .. 24 */
    uint32_t h = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (h & 1u))) ++h;
    return (uint16_t)(sign | h);
  }
  uint32_t h = ((exp - 112u) << 10) | ((ax & 0x7fffffu) >> 13);
  const uint32_t rem = ax & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) ++h; /* a carry moves into the exponent */
  return (uint16_t)(sign | h);
}

/* float -> bfloat16, round to nearest even (add-and-shift); NaN stays a quiet NaN. */
static uint16_t float_to_bf16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x0040u);
  return (uint16_t)((x + 0x7fffu + ((x >> 16) & 1u)) >> 16);
}

void oracle_f32_to_f16_bits(const float* x, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = float_to_half(x[i]);
}
void oracle_f32_to_bf16_bits(const float* x, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = float_to_bf16(x[i]);
}

/* Gradient dtypes: 0 = fp32, 1 = binary16, 2 = bfloat16; widening is exact, as group_cast's is
 * (python/raf/optim/lans.py:261-265). */
static inline double load_grad(const void* g, int g_dtype, int64_t i, float unscale) {
  float g32 = g_dtype == 1   ? half_to_float(((const uint16_t*)g)[i])
              : g_dtype == 2 ? bf16_to_float(((const uint16_t*)g)[i])
                             : ((const float*)g)[i];
  float scaled = g32 * unscale; /* one fp32 rounding, exact for powers of two */
  return (double)scaled;
}

#define ORACLE_BLOCK 4096

/* Blocked sums: each block is summed by one thread and the block partials are then added in
 * index order, so the result does not depend on the thread count. */
static double ordered_total(const double* part, int64_t nb) {
  double total = 0.0;
  for (int64_t b = 0; b < nb; ++b) total += part[b];
  return total;
}

static double sumsq_grad(const void* g, int g_dtype, int64_t n, float unscale, double* part) {
  int64_t nb = (n + ORACLE_BLOCK - 1) / ORACLE_BLOCK;
#pragma omp parallel for schedule(static) if (n > (1 << 16))
  for (int64_t b = 0; b < nb; ++b) {
    int64_t lo = b * ORACLE_BLOCK, hi = lo + ORACLE_BLOCK < n ? lo + ORACLE_BLOCK : n;
    double s = 0.0;
    for (int64_t i = lo; i < hi; ++i) {
      double x = load_grad(g, g_dtype, i, unscale);
      s += x * x;
    }
    part[b] = s;
  }
  return ordered_total(part, nb);
}

static double sumsq_f32(const float* a, int64_t n, double* part) {
  int64_t nb = (n + ORACLE_BLOCK - 1) / ORACLE_BLOCK;
#pragma omp parallel for schedule(static) if (n > (1 << 16))
  for (int64_t b = 0; b < nb; ++b) {
    int64_t lo = b * ORACLE_BLOCK, hi = lo + ORACLE_BLOCK < n ? lo + ORACLE_BLOCK : n;
    double s = 0.0;
    for (int64_t i = lo; i < hi; ++i) s += (double)a[i] * (double)a[i];
    part[b] = s;
  }
  return ordered_total(part, nb);
}

typedef struct {
  double lr, beta1, beta2, omb2, beta3, eps, wd, bc1, bc2;
} scalars_t;

static scalars_t make_scalars(const oracle_lans_hparams* hp, float step_value) {
  scalars_t s;
  int step = (int)step_value; /* lans.cc:98-99 */
  float bc1 = 1.0f, bc2 = 1.0f, beta3 = 1.0f;
  if (hp->bias_correction == 1) { /* lans.cc:102-105: double pow, stored in a float */
    bc1 = (float)(1.0 - pow((double)hp->beta1, (double)step));
    bc2 = (float)(1.0 - pow((double)hp->beta2, (double)step));
  }
  if (hp->grad_averaging == 1) { /* lans.cc:107-109: fp32 subtraction */
    volatile float b3 = 1.0f - hp->beta1;
    beta3 = b3;
  }
  volatile float omb2 = 1.0f - hp->beta2; /* multi_tensor_lans.cu:291 */
  s.lr = hp->learning_rate;
  s.beta1 = hp->beta1;
  s.beta2 = hp->beta2;
  s.omb2 = omb2;
  s.beta3 = beta3;
  s.eps = hp->eps;
  s.wd = hp->weight_decay;
  s.bc1 = bc1;
  s.bc2 = bc2;
  return s;
}

static inline void directions(double g, double w, double m, double v, const scalars_t* s,
                              int normalize, double gn, int mode, double* m1, double* v1,
                              double* um, double* ug) {
  double sg = g;
  if (normalize && gn != 0.0) sg = g / (gn + s->eps);
  double wp = (s->wd != 0.0) ? w : 0.0;
  if (mode == 0) sg = sg + s->wd * wp;
  double mn = m * s->beta1 + s->beta3 * sg;
  double vn = v * s->beta2 + s->omb2 * sg * sg;
  double den = sqrt(vn / s->bc2) + s->eps;
  if (mode == 0) {
    *um = (mn / s->bc1) / den;
    *ug = sg / den;
  } else {
    double sp = s->wd * wp;
    *um = (mn / s->bc1) / den + sp;
    *ug = sg / den + sp;
  }
  *m1 = mn;
  *v1 = vn;
}

/*
 * One LANS step over n tensors, in place on w/m/v (fp32 storage, float64 arithmetic).
 * g[t] points at numel[t] gradients of dtype g_dtype (0 fp32, 1 binary16, 2 bfloat16); g is not
 * modified.  If p is not NULL, p[t] receives the stored fp32 weight narrowed to p_dtype (1 binary16,
 * 2 bfloat16): the model's half-precision parameter (python/raf/optim/lans.py:289-291, :303-305).
 * norms_out, if not NULL, receives 4 doubles per tensor: ||g||, ||w||, ||u_m||, ||u_g||.
 */
void oracle_lans_step(int32_t n_tensors, const int64_t* numel, const void* const* g, int g_dtype,
                      float* const* w, float* const* m, float* const* v, float step_value,
                      const oracle_lans_hparams* hp, double* norms_out, int threads,
                      uint16_t* const* p, int p_dtype) {
  scalars_t s = make_scalars(hp, step_value);
#ifdef _OPENMP
  if (threads > 0) omp_set_num_threads(threads);
#else
  (void)threads;
#endif
  for (int32_t t = 0; t < n_tensors; ++t) {
    const int64_t n = numel[t];
    const void* gt = g[t];
    float *wt = w[t], *mt = m[t], *vt = v[t];
    const float us = hp->grad_unscale;
    int64_t nb = (n + ORACLE_BLOCK - 1) / ORACLE_BLOCK;
    double* part = (double*)malloc((size_t)(2 * nb + 2) * sizeof(double));
    double* part2 = part + nb + 1;
    const double gn = sqrt(sumsq_grad(gt, g_dtype, n, us, part));
    const double pn = sqrt(sumsq_f32(wt, n, part));

#pragma omp parallel for schedule(static) if (n > (1 << 16))
    for (int64_t b = 0; b < nb; ++b) {
      int64_t lo = b * ORACLE_BLOCK, hi = lo + ORACLE_BLOCK < n ? lo + ORACLE_BLOCK : n;
      double a = 0.0, c = 0.0;
      for (int64_t i = lo; i < hi; ++i) {
        double m1, v1, um, ug;
        directions(load_grad(gt, g_dtype, i, us), wt[i], mt[i], vt[i], &s, hp->normalize_grad, gn,
                   hp->mode, &m1, &v1, &um, &ug);
        a += um * um;
        c += ug * ug;
      }
      part[b] = a;
      part2[b] = c;
    }
    const double unm = sqrt(ordered_total(part, nb)), ung = sqrt(ordered_total(part2, nb));
    free(part);
    double rm = (unm != 0.0 && pn != 0.0) ? s.lr * (pn / unm) : s.lr;
    double rg = (ung != 0.0 && pn != 0.0) ? s.lr * (pn / ung) : s.lr;
    rm *= s.beta1;
    rg *= s.beta3;
#pragma omp parallel for schedule(static) if (n > (1 << 16))
    for (int64_t i = 0; i < n; ++i) {
      double m1, v1, um, ug;
      double w0 = wt[i];
      directions(load_grad(gt, g_dtype, i, us), w0, mt[i], vt[i], &s, hp->normalize_grad, gn,
                 hp->mode, &m1, &v1, &um, &ug);
      wt[i] = (float)(w0 - rm * um - rg * ug);
      if (p) p[t][i] = p_dtype == 2 ? float_to_bf16(wt[i]) : float_to_half(wt[i]);
      mt[i] = (float)m1;
      vt[i] = (float)v1;
    }
    if (norms_out) {
      norms_out[4 * t + 0] = gn;
      norms_out[4 * t + 1] = pn;
      norms_out[4 * t + 2] = unm;
      norms_out[4 * t + 3] = ung;
    }
  }
}

int oracle_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
