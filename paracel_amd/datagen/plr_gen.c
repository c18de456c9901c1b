/*
 * Seeded synthetic-shard generator for the logistic-regression benchmarks and
 * parity tests.  Host only: the device receives bytes, never a seed, so the
 * same (seed, shape) regenerates bit-identical shards on any box.
 *
 * Counter-based: element (i, j) of stream s is output j of a splitmix64
 * sequence whose state is keyed by (seed, s, i).  Uniforms come from exact
 * bit scaling, normals from Wichura's AS241 (PPND16) inverse CDF, which uses
 * only + * / and, in the tails, sqrt and log -- no std::normal_distribution,
 * whose output is implementation-defined.  Built with -ffp-contract=off.
 *
 * The reference's own LR inputs come from sklearn make_classification
 * (tool/datagen.py:73-75) written as CSV "f1,...,fk,label"; this generator
 * produces the same shape of data (dense rows, labels in {0,1}) directly in
 * the row-major fp64 layout the worker keeps after lr.cpp:76-93.
 */
#include "plr_gen.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>

#define GOLD 0x9E3779B97F4A7C15ULL

static inline uint64_t sm64_mix(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
  return z ^ (z >> 31);
}

static inline uint64_t row_key(uint64_t seed, uint64_t stream, uint64_t i) {
  return sm64_mix(sm64_mix(seed + stream * GOLD) + (i + 1) * GOLD);
}

static inline uint64_t elem_bits(uint64_t rk, uint64_t j) {
  return sm64_mix(rk + (j + 1) * GOLD);
}

/* (0,1), never 0 or 1: 53 bits + half an ulp. */
static inline double u01(uint64_t bits) {
  return ((double)(bits >> 11) + 0.5) * (1.0 / 9007199254740992.0);
}

/* Wichura (1988) Algorithm AS241, PPND16: inverse normal CDF, ~1e-16. */
static double ppnd16(double p) {
  static const double a[8] = {3.3871328727963666080e0, 1.3314166789178437745e+2,
      1.9715909503065514427e+3, 1.3731693765509461125e+4,
      4.5921953931549871457e+4, 6.7265770927008700853e+4,
      3.3430575583588128105e+4, 2.5090809287301226727e+3};
  static const double b[8] = {1.0, 4.2313330701600911252e+1,
      6.8718700749205790830e+2, 5.3941960214247511077e+3,
      2.1213794301586595867e+4, 3.9307895800092710610e+4,
      2.8729085735721942674e+4, 5.2264952788528545610e+3};
  static const double c[8] = {1.42343711074968357734e0, 4.63033784615654529590e0,
      5.76949722146069140550e0, 3.64784832476320460504e0,
      1.27045825245236838258e0, 2.41780725177450611770e-1,
      2.27238449892691845833e-2, 7.74545014278341407640e-4};
  static const double dd[8] = {1.0, 2.05319162663775882187e0,
      1.67638483018380384940e0, 6.89767334985100004550e-1,
      1.48103976427480074590e-1, 1.51986665636164571966e-2,
      5.47593808499534494600e-4, 1.05075007164441684324e-9};
  static const double e[8] = {6.65790464350110377720e0, 5.46378491116411436990e0,
      1.78482653991729133580e0, 2.96560571828504891230e-1,
      2.65321895265761230930e-2, 1.24266094738807843860e-3,
      2.71155556874348757815e-5, 2.01033439929228813265e-7};
  static const double f[8] = {1.0, 5.99832206555887937690e-1,
      1.36929880922735805310e-1, 1.48753612908506148525e-2,
      7.86869131145613259100e-4, 1.84631831751005468180e-5,
      1.42151175831644588870e-7, 2.04426310338993978564e-15};
  double q = p - 0.5, r, num, den;
  int k;
  if (fabs(q) <= 0.425) {
    r = 0.180625 - q * q;
    num = a[7]; den = b[7];
    for (k = 6; k >= 0; --k) { num = num * r + a[k]; den = den * r + b[k]; }
    return q * num / den;
  }
  r = (q < 0.0) ? p : 1.0 - p;
  r = sqrt(-log(r));
  if (r <= 5.0) {
    r -= 1.6;
    num = c[7]; den = dd[7];
    for (k = 6; k >= 0; --k) { num = num * r + c[k]; den = den * r + dd[k]; }
  } else {
    r -= 5.0;
    num = e[7]; den = f[7];
    for (k = 6; k >= 0; --k) { num = num * r + e[k]; den = den * r + f[k]; }
  }
  return (q < 0.0) ? -(num / den) : (num / den);
}

double plr_gen_u01(uint64_t seed, uint64_t stream, uint64_t i, uint64_t j) {
  return u01(elem_bits(row_key(seed, stream, i), j));
}

double plr_gen_normal(uint64_t seed, uint64_t stream, uint64_t i, uint64_t j) {
  return ppnd16(plr_gen_u01(seed, stream, i, j));
}

static void gen_rows(const plr_gen_spec* sp, int64_t row0, int64_t r_lo,
                     int64_t r_hi, int64_t d, int64_t ldx, double* X) {
  for (int64_t r = r_lo; r < r_hi; ++r) {
    uint64_t i = (uint64_t)(row0 + r);
    uint64_t rk = row_key(sp->seed, PLR_STREAM_X, i);
    uint64_t zk = row_key(sp->seed, PLR_STREAM_ZERO, i);
    double rs = 1.0;
    if (sp->outlier_mod > 0 &&
        row_key(sp->seed, PLR_STREAM_OUTLIER, i) % (uint64_t)sp->outlier_mod == 0)
      rs = sp->outlier_scale;
    double* x = X + r * ldx;
    for (int64_t j = 0; j < d; ++j) {
      double v;
      if (sp->zero_prob > 0.0 && u01(elem_bits(zk, (uint64_t)j)) < sp->zero_prob) {
        v = 0.0;
      } else {
        double u = u01(elem_bits(rk, (uint64_t)j));
        v = (sp->kind == PLR_GEN_UNIFORM) ? sp->scale * (2.0 * u - 1.0)
                                          : sp->scale * ppnd16(u);
        v *= rs;
      }
      x[j] = v;
    }
    for (int64_t j = d; j < ldx; ++j) x[j] = 0.0;
  }
}

typedef struct {
  const plr_gen_spec* sp; int64_t row0, lo, hi, d, ldx; double* X;
  const double* theta; double* y;
} job_t;

static void* gen_rows_thr(void* p) {
  job_t* j = (job_t*)p;
  gen_rows(j->sp, j->row0, j->lo, j->hi, j->d, j->ldx, j->X);
  return 0;
}

static void run_jobs(void* (*fn)(void*), job_t* proto, int64_t nrows,
                     int threads) {
  if (threads < 1) threads = 1;
  if (threads > 256) threads = 256;
  if (nrows < threads) threads = nrows > 0 ? (int)nrows : 1;
  pthread_t th[256];
  job_t jobs[256];
  for (int t = 0; t < threads; ++t) {
    jobs[t] = *proto;
    jobs[t].lo = nrows * t / threads;
    jobs[t].hi = nrows * (t + 1) / threads;
  }
  if (threads == 1) { fn(&jobs[0]); return; }
  for (int t = 0; t < threads; ++t) pthread_create(&th[t], 0, fn, &jobs[t]);
  for (int t = 0; t < threads; ++t) pthread_join(th[t], 0);
}

void plr_gen_X(const plr_gen_spec* sp, int64_t row0, int64_t nrows, int64_t d,
               int64_t ldx, double* X, int threads) {
  job_t j = {sp, row0, 0, nrows, d, ldx, X, 0, 0};
  run_jobs(gen_rows_thr, &j, nrows, threads);
}

void plr_gen_vec(uint64_t seed, uint64_t stream, int kind, double scale,
                 double nonzero_frac, int64_t n, double* out) {
  uint64_t rk = row_key(seed, stream, 0);
  uint64_t zk = row_key(seed, stream, 1);
  for (int64_t j = 0; j < n; ++j) {
    double u = u01(elem_bits(rk, (uint64_t)j));
    double v = (kind == PLR_GEN_UNIFORM) ? scale * (2.0 * u - 1.0)
                                         : scale * ppnd16(u);
    if (nonzero_frac < 1.0 && !(u01(elem_bits(zk, (uint64_t)j)) < nonzero_frac))
      v = 0.0;
    out[j] = v;
  }
}

static void* labels_thr(void* p) {
  job_t* jb = (job_t*)p;
  for (int64_t r = jb->lo; r < jb->hi; ++r) {
    const double* x = jb->X + r * jb->ldx;
    /* long double dot so the label does not depend on a summation order */
    long double z = 0.0L;
    for (int64_t j = 0; j < jb->d; ++j)
      z += (long double)x[j] * (long double)jb->theta[j];
    double p1 = (double)(1.0L / (1.0L + expl(-z)));
    double u = plr_gen_u01(jb->sp->seed, PLR_STREAM_LABEL,
                           (uint64_t)(jb->row0 + r), 0);
    jb->y[r] = (u < p1) ? 1.0 : 0.0;
  }
  return 0;
}

void plr_gen_labels(const plr_gen_spec* sp, int64_t row0, int64_t nrows,
                    int64_t d, int64_t ldx, const double* X,
                    const double* theta_star, double* y, int threads) {
  job_t j = {sp, row0, 0, nrows, d, ldx, (double*)X, theta_star, y};
  run_jobs(labels_thr, &j, nrows, threads);
}
