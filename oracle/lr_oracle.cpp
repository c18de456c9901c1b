/*
 * CPU oracle for Paracel's worker-side logistic-regression arithmetic.
 * TEST INFRASTRUCTURE ONLY -- see lr_oracle.h for what may use it, what each
 * function restates (reference file:line) and how it is pinned.
 *
 * Build: g++ -O3 -ffp-contract=off (generic x86-64: no FMA, as the
 * reference's own -O3 -std=c++11 build, CMakeLists.txt:9-11).
 */
#include "lr_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <chrono>
#include <functional>
#include <numeric>
#include <string>
#include <thread>
#include <vector>

using std::vector;

namespace {

/* The reference keeps each sample as its own std::vector<double>
 * (lr.hpp:75); the flat-array entry points below view rows in place so that
 * tests need no copies, while the baseline timer builds the real layout. */
inline double dot_seq(const double* a, const double* b, int64_t d) {
  /* std::inner_product(a.begin(), a.end(), b.begin(), 0.) */
  return std::inner_product(a, a + d, b, 0.);
}

inline double hypothesis(const double* x, const double* theta, int64_t d) {
  double dp = dot_seq(x, theta, d);
  return 1. / (1. + exp(-dp));
}

inline long double dot_hp(const double* a, const double* b, int64_t d) {
  long double s = 0.L;
  for (int64_t j = 0; j < d; ++j) s += (long double)a[j] * (long double)b[j];
  return s;
}

inline long double hypothesis_hp(const double* x, const double* theta,
                                 int64_t d) {
  return 1.L / (1.L + expl(-dot_hp(x, theta, d)));
}

}  // namespace

extern "C" {

double oracle_dot_product(const double* a, const double* b, int64_t d) {
  return dot_seq(a, b, d);
}

double oracle_lr_hypothesis(const double* x, const double* theta, int64_t d) {
  return hypothesis(x, theta, d);
}

void oracle_dgd_delta(const double* X, int64_t n, int64_t d, int64_t ldx,
                      const double* y, const double* theta, double alpha,
                      double beta, const int64_t* order, double* delta) {
  double coff2 = 2. * beta * alpha;
  for (int64_t i = 0; i < d; ++i) delta[i] = 0.;
  for (int64_t k = 0; k < n; ++k) {
    int64_t sample_id = order ? order[k] : k;
    const double* x = X + sample_id * ldx;
    double grad = y[sample_id] - hypothesis(x, theta, d);
    double coff1 = alpha * grad;
    for (int64_t i = 0; i < d; ++i) {
      double t = coff1 * x[i] - coff2 * theta[i];
      delta[i] += t;
    }
  }
}

double oracle_calc_loss_sum(const double* X, int64_t n, int64_t d, int64_t ldx,
                            const double* y, const double* theta) {
  double loss = 0.;
  for (int64_t i = 0; i < n; ++i) {
    double h = hypothesis(X + i * ldx, theta, d);
    if (y[i] == 1.) {
      loss += -log(h);
    } else {
      loss += -log(1 - h);
    }
  }
  return loss;
}

double oracle_calc_loss(const double* X, int64_t n, int64_t d, int64_t ldx,
                        const double* y, const double* theta) {
  return oracle_calc_loss_sum(X, n, d, ldx, y, theta) /
         static_cast<double>(n);
}

void oracle_theta_update(const double* a, const double* b, int64_t d,
                         double* r) {
  for (int64_t i = 0; i < d; ++i) r[i] = a[i] + b[i];
}

void oracle_predict(const double* X, int64_t n, int64_t d, int64_t ldx,
                    const double* theta, double* h_out) {
  for (int64_t i = 0; i < n; ++i) h_out[i] = hypothesis(X + i * ldx, theta, d);
}

void oracle_gsum(const double* X, int64_t n, int64_t d, int64_t ldx,
                 const double* y, const double* theta, double* gsum) {
  for (int64_t j = 0; j < d; ++j) gsum[j] = 0.;
  for (int64_t i = 0; i < n; ++i) {
    const double* x = X + i * ldx;
    double r = hypothesis(x, theta, d) - y[i];
    for (int64_t j = 0; j < d; ++j) gsum[j] += r * x[j];
  }
}

void oracle_train_dgd(const double* X, int64_t n, int64_t d, int64_t ldx,
                      const double* y, double* theta, double alpha,
                      double beta, int rounds) {
  vector<double> delta(d);
  for (int rd = 0; rd < rounds; ++rd) {
    oracle_dgd_delta(X, n, d, ldx, y, theta, alpha, beta, nullptr,
                     delta.data());
    for (int64_t i = 0; i < d; ++i) theta[i] += delta[i];
  }
}

void oracle_train_dgd_workers(const double* X, int64_t n, int64_t d, int64_t ldx,
                              const double* y, double* theta, double alpha,
                              double beta, int rounds, int workers) {
  if (workers < 1) workers = 1;
  vector<vector<double> > delta(workers, vector<double>(d));
  for (int rd = 0; rd < rounds; ++rd) {
    vector<std::thread> th;
    for (int w = 0; w < workers; ++w) {
      const int64_t lo = n * w / workers, hi = n * (w + 1) / workers;
      th.emplace_back([=, &delta]() {
        oracle_dgd_delta(X + lo * ldx, hi - lo, d, ldx, y + lo, theta, alpha, beta,
                         nullptr, delta[w].data());
      });
    }
    for (auto& t : th) t.join();
    for (int w = 0; w < workers; ++w)
      for (int64_t i = 0; i < d; ++i) theta[i] = theta[i] + delta[w][i];
  }
}

int64_t oracle_local_parser(const char* text, int64_t nlines, char sep,
                            double* X_out, double* y_out,
                            int64_t k_expected) {
  const char* p = text;
  int64_t D = -1;
  for (int64_t ln = 0; ln < nlines; ++ln) {
    const char* eol = strchr(p, '\n');
    if (!eol) eol = p + strlen(p);
    /* split on sep; every field but the last is a feature, the last the
     * label; a leading 1.0 is the bias column. */
    vector<double> fields;
    const char* q = p;
    while (q <= eol) {
      const char* e = q;
      while (e < eol && *e != sep) ++e;
      std::string tok(q, e);
      if (!tok.empty()) { /* str_split drops empty fields
                             (include/utils/ext_utility.hpp:38-50) */
        char* endp = nullptr;
        double v = strtod(tok.c_str(), &endp); /* std::stod wraps strtod */
        if (endp == tok.c_str()) return -1;    /* std::stod would throw */
        fields.push_back(v);
      }
      q = e + 1;
    }
    int64_t k = (int64_t)fields.size() - 1;
    if (k < 0) return -1;
    if (D < 0) {
      D = k + 1;
      if (k_expected >= 0 && k != k_expected) return -1;
    } else if (k + 1 != D) {
      return -1;
    }
    double* row = X_out + ln * D;
    row[0] = 1.;
    for (int64_t i = 0; i < k; ++i) row[i + 1] = fields[i];
    y_out[ln] = fields.back();
    p = (*eol == '\n') ? eol + 1 : eol;
  }
  return D;
}

double oracle_ridge_loss_sum(const double* X, int64_t n, int64_t d, int64_t ldx,
                             const double* y, const double* theta) {
  double loss = 0.;
  for (int64_t i = 0; i < n; ++i) {
    double h = dot_seq(X + i * ldx, theta, d) - y[i];
    loss += h * h;
  }
  return loss;
}

void oracle_predict_linear(const double* X, int64_t n, int64_t d, int64_t ldx,
                           const double* theta, double* z_out) {
  for (int64_t i = 0; i < n; ++i) z_out[i] = dot_seq(X + i * ldx, theta, d);
}

void oracle_lsq_gsum(const double* X, int64_t n, int64_t d, int64_t ldx,
                     const double* y, const double* theta, double* gsum) {
  for (int64_t j = 0; j < d; ++j) gsum[j] = 0.;
  for (int64_t i = 0; i < n; ++i) {
    const double* x = X + i * ldx;
    double r = dot_seq(x, theta, d) - y[i];
    for (int64_t j = 0; j < d; ++j) gsum[j] += r * x[j];
  }
}

void oracle_ridge_delta(const double* X, int64_t n, int64_t d, int64_t ldx,
                        const double* y, const double* theta, double alpha,
                        double beta, double* delta) {
  const double coff2 = 2. * beta * alpha;
  for (int64_t i = 0; i < d; ++i) delta[i] = 0.;
  for (int64_t k = 0; k < n; ++k) {
    const double* x = X + k * ldx;
    const double coff1 = alpha * (y[k] - dot_seq(x, theta, d));
    for (int64_t i = 0; i < d; ++i) {
      double t = coff1 * x[i] - coff2 * theta[i];
      delta[i] += t;
    }
  }
}

void oracle_ridge_train_workers(const double* X, int64_t n, int64_t d, int64_t ldx,
                                const double* y, double* theta, double alpha,
                                double beta, int rounds, int workers) {
  if (workers < 1) workers = 1;
  vector<vector<double> > delta(workers, vector<double>(d));
  for (int rd = 0; rd < rounds; ++rd) {
    for (int w = 0; w < workers; ++w) {
      const int64_t lo = n * w / workers, hi = n * (w + 1) / workers;
      oracle_ridge_delta(X + lo * ldx, hi - lo, d, ldx, y + lo, theta, alpha, beta,
                         delta[w].data());
    }
    for (int w = 0; w < workers; ++w)
      for (int64_t i = 0; i < d; ++i) theta[i] = theta[i] + delta[w][i];
  }
}

void oracle_gsum_hp(const double* X, int64_t n, int64_t d, int64_t ldx,
                    const double* y, const double* theta, double* gsum) {
  vector<long double> acc(d, 0.L);
  for (int64_t i = 0; i < n; ++i) {
    const double* x = X + i * ldx;
    long double r = hypothesis_hp(x, theta, d) - (long double)y[i];
    for (int64_t j = 0; j < d; ++j) acc[j] += r * (long double)x[j];
  }
  for (int64_t j = 0; j < d; ++j) gsum[j] = (double)acc[j];
}

void oracle_dgd_delta_hp(const double* X, int64_t n, int64_t d, int64_t ldx,
                         const double* y, const double* theta, double alpha,
                         double beta, double* delta) {
  long double coff2 = 2.L * (long double)beta * (long double)alpha;
  vector<long double> acc(d, 0.L);
  for (int64_t k = 0; k < n; ++k) {
    const double* x = X + k * ldx;
    long double coff1 =
        (long double)alpha * ((long double)y[k] - hypothesis_hp(x, theta, d));
    for (int64_t i = 0; i < d; ++i)
      acc[i] += coff1 * (long double)x[i] - coff2 * (long double)theta[i];
  }
  for (int64_t i = 0; i < d; ++i) delta[i] = (double)acc[i];
}

double oracle_calc_loss_sum_hp(const double* X, int64_t n, int64_t d,
                               int64_t ldx, const double* y,
                               const double* theta) {
  long double loss = 0.L;
  for (int64_t i = 0; i < n; ++i) {
    long double h = hypothesis_hp(X + i * ldx, theta, d);
    loss += (y[i] == 1.) ? -logl(h) : -logl(1.L - h);
  }
  return (double)loss;
}

double oracle_stable_loss_sum_hp(const double* X, int64_t n, int64_t d,
                                 int64_t ldx, const double* y,
                                 const double* theta) {
  long double loss = 0.L;
  for (int64_t i = 0; i < n; ++i) {
    long double z = dot_hp(X + i * ldx, theta, d);
    long double s = (y[i] == 1.) ? -z : z; /* loss = log(1+exp(s)) */
    loss += log1pl(expl(-fabsl(s))) + (s > 0.L ? s : 0.L);
  }
  return (double)loss;
}

double oracle_baseline_time(const double* X, int64_t n, int64_t d, int64_t ldx,
                            const double* y, const double* theta_in,
                            double alpha, double beta, int threads, int reps,
                            double* delta_out, double* loss_seconds,
                            double* loss_sum) {
  if (threads < 1) threads = 1;
  if (reps < 1) reps = 1;
  struct shard {
    vector<vector<double> > samples;
    vector<double> labels;
    vector<double> theta;
    vector<double> delta;
    double loss = 0.;
  };
  vector<shard> sh(threads);
  auto fill = [&](int t) {
    int64_t lo = n * t / threads, hi = n * (t + 1) / threads;
    shard& s = sh[t];
    s.samples.reserve(hi - lo);
    for (int64_t i = lo; i < hi; ++i) {
      const double* x = X + i * ldx;
      s.samples.push_back(vector<double>(x, x + d));
      s.labels.push_back(y[i]);
    }
    s.theta.assign(theta_in, theta_in + d);
    s.delta.assign(d, 0.);
  };
  auto traverse = [&](int t) {
    shard& s = sh[t];
    const vector<double>& theta = s.theta;
    vector<double>& delta = s.delta;
    int data_dim = (int)d;
    double coff2 = 2. * beta * alpha;
    for (int i = 0; i < data_dim; ++i) delta[i] = 0.;
    for (size_t sample_id = 0; sample_id < s.samples.size(); ++sample_id) {
      const vector<double>& v = s.samples[sample_id];
      double dp = std::inner_product(v.begin(), v.end(), theta.begin(), 0.);
      double grad = s.labels[sample_id] - 1. / (1. + exp(-dp));
      double coff1 = alpha * grad;
      for (int i = 0; i < data_dim; ++i) {
        double t2 = coff1 * v[i] - coff2 * theta[i];
        delta[i] += t2;
      }
    }
  };
  auto lossf = [&](int t) {
    shard& s = sh[t];
    double loss = 0.;
    for (size_t i = 0; i < s.samples.size(); ++i) {
      const vector<double>& v = s.samples[i];
      double dp = std::inner_product(v.begin(), v.end(), s.theta.begin(), 0.);
      double h = 1. / (1. + exp(-dp));
      if (s.labels[i] == 1.) loss += -log(h);
      else loss += -log(1 - h);
    }
    s.loss = loss;
  };
  auto run_all = [&](const std::function<void(int)>& f) {
    if (threads == 1) { f(0); return; }
    vector<std::thread> th;
    for (int t = 0; t < threads; ++t) th.emplace_back(f, t);
    for (auto& x : th) x.join();
  };
  run_all(fill);
  auto t0 = std::chrono::steady_clock::now();
  for (int r = 0; r < reps; ++r) run_all(traverse);
  auto t1 = std::chrono::steady_clock::now();
  double sec = std::chrono::duration<double>(t1 - t0).count() / reps;
  if (delta_out) {
    /* the server folds worker deltas one at a time: theta + d0 + d1 + ...
     * (update.cpp:26-32); the sum of deltas in worker order is the part of
     * that which does not depend on theta. */
    for (int64_t i = 0; i < d; ++i) {
      double acc = sh[0].delta[i];
      for (int t = 1; t < threads; ++t) acc = acc + sh[t].delta[i];
      delta_out[i] = acc;
    }
  }
  if (loss_seconds || loss_sum) {
    auto t2 = std::chrono::steady_clock::now();
    run_all(lossf);
    auto t3 = std::chrono::steady_clock::now();
    if (loss_seconds) *loss_seconds = std::chrono::duration<double>(t3 - t2).count();
    if (loss_sum) {
      double acc = 0.;
      for (int t = 0; t < threads; ++t) acc += sh[t].loss;
      *loss_sum = acc;
    }
  }
  return sec;
}

}  // extern "C"
