/*
 * CPU oracle for Paracel's worker-side logistic-regression arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker the HIP path is
 * compared against; nothing in the shipped product (libplr.so, the worker
 * classes) links, loads or calls it.  Only tests/, __graft_entry__.smoke()
 * and bench.py's cpu_baseline leg may use it.
 *
 * Each function restates a few lines of the reference (cited per function)
 * in the reference's own evaluation order: fp64, strictly sequential sums,
 * no FMA contraction (built with -ffp-contract=off for generic x86-64, as
 * the reference's -O3 build is).  The *_hp twins carry every sum in
 * long double (x87 80-bit) and are used to arbitrate rounding disputes.
 *
 * Parity status: the reference ships no test, fixture or golden vector for
 * any of these functions (its test/ directory never names lr.cpp, lr_serial,
 * dot_product, lr_hypothesis, calc_loss or local_update), and the reference
 * cannot be compiled in this image (ps.hpp needs Boost, Eigen3, msgpack-c,
 * gflags; none installed).  The oracle is therefore pinned by mathematics:
 * closed forms (theta = 0, X = 0, one-hot rows), library routines (numpy
 * GEMV, scipy expit/log1p), exact-rational brute force on tiny inputs,
 * symmetry and additivity invariants -- see tests/test_oracle_pins.py.
 */
#ifndef PLR_LR_ORACLE_H
#define PLR_LR_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* include/utils/ext_utility.hpp:171-174 -- std::inner_product from 0.0,
 * strict left-to-right. */
double oracle_dot_product(const double* a, const double* b, int64_t d);

/* alg/classification/logistic_regression/lr.cpp:69-72 (twin
 * tool/lr_serial.cpp:65-68): 1/(1+exp(-x.theta)), no clamping. */
double oracle_lr_hypothesis(const double* x, const double* theta, int64_t d);

/* lr.cpp:119,125-127,132-138 (twin tool/lr_serial.cpp:95-104): one round's
 * delta.  coff2 = 2*beta*alpha; delta = 0; for each row in `order` (identity
 * when order == NULL; the reference shuffles with a time seed, which only
 * permutes the rounding): coff1 = alpha*(y - h);
 * t = coff1*x[i] - coff2*theta[i]; delta[i] += t. */
void oracle_dgd_delta(const double* X, int64_t n, int64_t d, int64_t ldx,
                      const double* y, const double* theta,
                      double alpha, double beta, const int64_t* order,
                      double* delta);

/* lr.cpp:322-330 (twin tool/lr_serial.cpp:126-135): sum over rows of
 * -log(h) when label == 1.0 exactly, else -log(1-h); row order, from 0.0.
 * This is the local sum before the two all-reduces of lr.cpp:331-334. */
double oracle_calc_loss_sum(const double* X, int64_t n, int64_t d, int64_t ldx,
                            const double* y, const double* theta);

/* lr.cpp:335: loss_sum / n_total. */
double oracle_calc_loss(const double* X, int64_t n, int64_t d, int64_t ldx,
                        const double* y, const double* theta);

/* alg/classification/logistic_regression/update.cpp:26-32: r[i]=a[i]+b[i]. */
void oracle_theta_update(const double* a, const double* b, int64_t d,
                         double* r);

/* lr.cpp:361-363: h per row, no reduction. */
void oracle_predict(const double* X, int64_t n, int64_t d, int64_t ldx,
                    const double* theta, double* h_out);

/* The quantity the device kernel returns: gsum = X^T (h - y), accumulated
 * row by row in fp64 (gsum[j] += (h_i - y_i) * x_ij), with h from
 * oracle_lr_hypothesis.  Related to oracle_dgd_delta by
 * delta = -alpha*gsum - 2*alpha*beta*n*theta in exact arithmetic
 * (lr.cpp:134-137 expanded). */
void oracle_gsum(const double* X, int64_t n, int64_t d, int64_t ldx,
                 const double* y, const double* theta, double* gsum);

/* tool/lr_serial.cpp:95-110: `rounds` full-batch iterations in place,
 * theta += delta after each traverse (identical to one worker against the
 * lr_theta_update reducer: lr.cpp:129-144 + update.cpp:26-32). */
void oracle_train_dgd(const double* X, int64_t n, int64_t d, int64_t ldx,
                      const double* y, double* theta,
                      double alpha, double beta, int rounds);

/* The same rounds with P local workers (mpirun -n P bin/lr, prun.py:78-79):
 * rows split into P contiguous shards, each worker traverses its shard
 * (lr.cpp:132-138) in its own thread, then the server folds the worker deltas
 * into theta one at a time in worker order (update.cpp:26-32 applied P times
 * per round).  P = 1 is oracle_train_dgd. */
void oracle_train_dgd_workers(const double* X, int64_t n, int64_t d, int64_t ldx,
                              const double* y, double* theta, double alpha,
                              double beta, int rounds, int workers);

/* lr.cpp:76-93: parse CSV lines "f1,...,fk,label" into rows [1.0,f1..fk]
 * and labels.  `text` holds `nlines` '\n'-separated lines.  X_out must hold
 * nlines*(k+1) doubles, y_out nlines.  Returns k+1 (row width D), or -1 on a
 * ragged/unparsable line. */
int64_t oracle_local_parser(const char* text, int64_t nlines, char sep,
                            double* X_out, double* y_out, int64_t k_expected);

/* alg/regression/ridge/ridge.hpp:103-109: sum over rows of (x.theta - y)^2,
 * row order, from 0.0 (the local sum before the all-reduces of :110-113). */
double oracle_ridge_loss_sum(const double* X, int64_t n, int64_t d, int64_t ldx,
                             const double* y, const double* theta);
/* ridge.hpp:130-139: x_i.theta per row. */
void oracle_predict_linear(const double* X, int64_t n, int64_t d, int64_t ldx,
                           const double* theta, double* z_out);
/* least-squares counterpart of oracle_gsum: X^T (X theta - y), row by row. */
void oracle_lsq_gsum(const double* X, int64_t n, int64_t d, int64_t ldx,
                     const double* y, const double* theta, double* gsum);

/* The ridge worker's update expression (ridge.hpp:79-84: coff1 = alpha*(y -
 * x.theta); t = coff1*x[i] - coff2*theta[i], coff2 = 2*beta*alpha) summed over
 * the rows at a FIXED theta: delta[i] += t, row order, from 0.0.  This is the
 * full-batch form of that expression (what lr.cpp:132-138 is for logistic
 * regression); the reference's own ridge trainer instead adds t to theta
 * inside the row loop (ridge.hpp:78-86) and is not restated here. */
void oracle_ridge_delta(const double* X, int64_t n, int64_t d, int64_t ldx,
                        const double* y, const double* theta, double alpha,
                        double beta, double* delta);
/* `rounds` rounds of that batch delta with P workers over contiguous row
 * shards and the server-side add of update.cpp:26-32 (ridge's update.cpp is
 * the same element-wise sum), in worker order. */
void oracle_ridge_train_workers(const double* X, int64_t n, int64_t d, int64_t ldx,
                                const double* y, double* theta, double alpha,
                                double beta, int rounds, int workers);

/* long-double arbiters: same formulas, every sum and exp/log in 80-bit. */
void oracle_gsum_hp(const double* X, int64_t n, int64_t d, int64_t ldx,
                    const double* y, const double* theta, double* gsum);
void oracle_dgd_delta_hp(const double* X, int64_t n, int64_t d, int64_t ldx,
                         const double* y, const double* theta,
                         double alpha, double beta, double* delta);
double oracle_calc_loss_sum_hp(const double* X, int64_t n, int64_t d,
                               int64_t ldx, const double* y,
                               const double* theta);
/* Stable loss: sum of log(1+exp(-|z|)) + max(-z,0) for y==1, +max(z,0) else;
 * long double.  Finite where the reference formula overflows to inf. */
double oracle_stable_loss_sum_hp(const double* X, int64_t n, int64_t d,
                                 int64_t ldx, const double* y,
                                 const double* theta);

/*
 * CPU baseline timer (bench.py's cpu_baseline leg only).  Copies rows
 * [0, n) into the reference's own layout -- std::vector<std::vector<double>>
 * samples, std::vector<double> labels (lr.hpp:75-76) -- split into `threads`
 * contiguous shards the way `mpirun -n P bin/lr` shards rows
 * (prun.py:78-79), then times `reps` traversals of lr.cpp:132-138 per shard
 * in parallel threads and sums the shard deltas as update.cpp:26-32 does.
 * Returns seconds per traversal (wall, max over shards); writes the summed
 * delta of the last rep.  loss_seconds (nullable) receives the time of one
 * calc_loss pass (lr.cpp:322-330) and loss_sum (nullable) its value.
 */
double oracle_baseline_time(const double* X, int64_t n, int64_t d, int64_t ldx,
                            const double* y, const double* theta,
                            double alpha, double beta, int threads, int reps,
                            double* delta_out, double* loss_seconds,
                            double* loss_sum);

#ifdef __cplusplus
}
#endif
#endif
