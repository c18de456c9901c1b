/*
 * plr -- C ABI of the MI355X logistic-regression shard kernels.
 *
 * A worker keeps its local shard (samples X, labels y) resident in HBM and,
 * once per round, hands over theta and receives the shard's loss and batch
 * gradient.  These entry points replace the inline loops of the reference's
 * worker (the reference has no FFI/plugin interface around this compute; the
 * loops sit between paracel_read and paracel_bupdate inside
 * logistic_regression::dgd_learning), so each declaration cites the
 * reference lines whose result it returns.
 *
 * Conventions: plain C types only; every pointer is caller-owned HOST memory,
 * valid for the duration of the call; calls are synchronous (they return
 * after the context's stream has drained); one context per worker process,
 * not thread-safe (as the reference's kvclt is not); results are bitwise
 * reproducible for a fixed (n, d, device).  All functions returning int give
 * PLR_OK (0) or a negative plr_status; plr_last_error() describes the last
 * failure on that context.
 */
#ifndef PLR_H
#define PLR_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct plr_ctx plr_ctx; /* opaque: device buffers + one HIP stream */

typedef enum {
  PLR_OK = 0,
  PLR_ERR_INVALID = -1,     /* null pointer, bad shape, bad flag            */
  PLR_ERR_HIP = -2,         /* a HIP runtime call failed                    */
  PLR_ERR_NOMEM = -3,       /* device or pinned allocation failed           */
  PLR_ERR_NODATA = -4,      /* no shard resident yet                        */
  PLR_ERR_UNSUPPORTED = -5  /* device is not a gfx950 part                  */
} plr_status;

/* loss formula selector for plr_loss_grad / plr_calc_loss */
#define PLR_LOSS_REFERENCE 0u /* -log(h) / -log(1-h): lr.cpp:325-329; may be
                                 +inf for saturated rows, like the reference */
#define PLR_LOSS_STABLE 1u    /* log1p(exp(-|z|)) + max(-/+z, 0): same value,
                                 finite for any z                            */
#define PLR_LOSS_NONE 2u      /* skip the loss (loss_sum receives 0)         */
#define PLR_LOSS_SQUARED 3u   /* linear model instead of logistic: residual
                                 x.theta - y, loss (x.theta - y)^2 -- the
                                 ridge worker's calc_loss,
                                 alg/regression/ridge/ridge.hpp:103-109       */

/* Create a context on HIP device `device_id`.  Replaces nothing in the
 * reference (which has no device); it is the constructor-time set-up a
 * worker does next to paralg's (include/ps.hpp:102-125). */
int plr_create(plr_ctx** out, int device_id);
void plr_destroy(plr_ctx* ctx);

/* Make the shard resident: n rows of d doubles, row-major with pitch
 * ldx >= d (in doubles), plus n labels.  Copies; the caller keeps its
 * buffers.  This is the layout lr.cpp:76-93 (local_parser) produces in
 * `samples`/`labels` (lr.hpp:75-76), flattened.  n may be 0. */
int plr_set_data(plr_ctx* ctx, const double* X, int64_t n, int64_t d,
                 int64_t ldx, const double* y);

/* Streaming form of the same: reserve an n x d shard (zero-filled), then fill
 * row ranges in any order; rows never sent stay zero rows with label 0.
 * ldx is the caller's row pitch, as in plr_set_data. */
int plr_alloc_data(plr_ctx* ctx, int64_t n, int64_t d);
int plr_set_data_chunk(plr_ctx* ctx, int64_t row0, int64_t nrows,
                       const double* X, int64_t ldx, const double* y);

/* The same from the sample text itself: local_parser (lr.cpp:76-93) on the
 * device.  text[0..nspans) / len[] are the worker's pieces of the input (the
 * lines paracel_load hands it, lr.cpp:303, as they lie in the files), every
 * non-empty line "f1<sep>f2<sep>...<sep>fk<sep>label".  The resident shard is
 * what local_parser builds -- the sample [1.0, f1..fk] (d = k + 1 columns,
 * *d_out) and the label -- with every field's value exactly std::stod's: the
 * device converts decimal spellings of up to 19 significant digits whose
 * correctly rounded value it can establish (all but those within 2^-30 of a
 * unit in the last place of a rounding tie; blanks and tabs in front are
 * skipped, a blank, a tab or the carriage return of a CR LF line end behind
 * the number ends it, as for std::stod), the rest (longer digit strings,
 * exponents beyond +-44, inf, nan, hex, a plus sign, other trailing
 * characters) are converted by std::stod on the host.  Empty fields are
 * skipped like the reference's str_split does.  *n_out receives the number
 * of samples.  Errors as the reference's parser would raise them (a field
 * std::stod rejects, a line with another number of fields) come back as
 * PLR_ERR_INVALID with the line number; lines of a single field are refused
 * with PLR_ERR_UNSUPPORTED.  The text is copied; the caller keeps it.
 * (plr_get_timing's last_ms afterwards: the duration of the parsing kernel;
 * for a text parsed while it arrived, option "csv_overlap", the time from the
 * first stretch's kernels to the last one's.) */
int plr_set_data_csv(plr_ctx* ctx, const char* const* text, const int64_t* len,
                     int nspans, char sep, int64_t* n_out, int64_t* d_out);

/* Rows row0 .. row0+nrows-1 of the resident shard back in the form
 * plr_set_data takes (row-major, pitch ldx >= d; X or y may be NULL): what a
 * worker needs to write its binary shard cache after plr_set_data_csv.  No
 * counterpart in the reference. */
int plr_get_data(plr_ctx* ctx, int64_t row0, int64_t nrows, double* X,
                 int64_t ldx, double* y);

/* One fused pass over the shard with theta (d doubles):
 *   gsum[j]  = sum_i (h_i - y_i) * x_ij,  h_i = 1/(1+exp(-x_i.theta))
 *              (lr.cpp:69-72 with ext_utility.hpp:171-174; the data term of
 *               lr.cpp:133-137 with the sign of the residual flipped and
 *               alpha factored out)
 *   loss_sum = sum_i l_i as lr.cpp:322-330 accumulates it (before the
 *              all-reduce and the division of lr.cpp:331-335)
 *   n_out    = number of rows summed.
 * gsum, loss_sum, n_out may each be NULL. */
int plr_loss_grad(plr_ctx* ctx, const double* theta, double* gsum,
                  double* loss_sum, int64_t* n_out, unsigned flags);

/* One round's delta exactly as lr.cpp:119,125-138 leaves it in `delta`
 * (reference signs): delta = alpha*X^T(y-h) - 2*alpha*beta*n*theta.
 * loss_sum (nullable) as above with the reference formula. */
int plr_dgd_delta(plr_ctx* ctx, const double* theta, double alpha, double beta,
                  double* delta, double* loss_sum);

/* The same round for the linear model (identity link instead of the sigmoid):
 * delta = alpha*X^T(y - X theta) - 2*alpha*beta*n*theta, i.e. the update
 * expression of the ridge worker, alg/regression/ridge/ridge.hpp:79-84
 * (coff1 = alpha*(y - x.theta); t = coff1*x[i] - coff2*theta[i]), summed over
 * the shard at a FIXED theta.  The reference's ridge trainer applies that
 * expression sample by sample, changing theta inside the row loop
 * (ridge.hpp:78-86); this is its full-batch form, as lr.cpp:132-138 is for
 * logistic regression.  loss_sum (nullable) receives sum_i (x_i.theta - y_i)^2
 * (ridge.hpp:103-109). */
int plr_dgd_delta_linear(plr_ctx* ctx, const double* theta, double alpha, double beta,
                         double* delta, double* loss_sum);

/* `rounds` full-batch rounds with theta kept on the device: each round is
 * lr.cpp:125-138 (delta at the current theta) followed by the reducer's
 * theta += delta (update.cpp:26-32) -- the single-process training loop of
 * tool/lr_serial.cpp:95-110, without a host round trip per round.  theta is
 * read at entry and overwritten with the result.  loss_curve (nullable,
 * `rounds` doubles) receives the loss sum (lr.cpp:322-330) at the theta each
 * round STARTED from.  With a parameter server in the loop use plr_dgd_delta
 * per round instead. */
int plr_train_dgd(plr_ctx* ctx, double* theta, double alpha, double beta, int rounds,
                  double* loss_curve);

/* lr.cpp:322-330: the loss pass alone (no gradient). */
int plr_calc_loss(plr_ctx* ctx, const double* theta, double* loss_sum,
                  int64_t* n_out, unsigned flags);

/* lr.cpp:361-363: h_i for every resident row (n doubles out). */
int plr_predict(plr_ctx* ctx, const double* theta, double* h_out);

/* alg/regression/ridge/ridge.hpp:130-139: x_i.theta for every resident row
 * (the linear model's prediction; n doubles out). */
int plr_predict_linear(plr_ctx* ctx, const double* theta, double* z_out);

/* plr_loss_grad for callers that cannot allocate device memory: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * No counterpart in the reference.  It needs no context and calls no
 * hipMalloc / hipFree: the caller passes every input and output as DEVICE
 * pointers, and the pass keeps its partial results (the zero-padded copy of
 * theta, the per-workgroup gradient and loss partials) in one static device
 * array of 8 MiB + 20 KiB per GPU, which that GPU holds until the process ends.
 *   dX     n rows at a pitch of ldx doubles; ldx must be a multiple of 128
 *          with d <= ldx <= 2048 (the limit of the static array; wider rows
 *          are refused with PLR_ERR_INVALID), columns d..ldx-1 must be zero
 *   dy     n labels;   dtheta  d doubles
 *   dout   d + 1 doubles: gsum as plr_loss_grad defines it, then loss_sum
 *   flags  a PLR_LOSS_* value
 * dX must be 16-byte aligned (the pass loads 16 bytes per lane), the other
 * pointers 8-byte aligned.
 * The work is enqueued on `hip_stream` (a hipStream_t; NULL = the default
 * stream) and the call returns without waiting: dout is valid once the stream
 * has reached that point.  All calls on one GPU share that GPU's static array,
 * so calls that may overlap on a GPU (different streams, different threads)
 * race; order them on one stream.
 * The first call on a device looks up the device's address of the static array
 * and its compute units, and the first call with a given ldx on a device asks
 * the runtime for that kernel's occupancy; both are remembered.  These
 * look-ups are not stream work: a caller that captures a stream makes one
 * call per ldx it will use BEFORE the capture begins; the captured calls then
 * only enqueue kernels (no memset or copy commands).  The caller's current
 * device is left as it was found.  Errors are described by
 * plr_last_error(NULL). */
int plr_loss_grad_noalloc(int device_id, void* hip_stream, const double* dX,
                          const double* dy, int64_t n, int64_t d, int64_t ldx,
                          const double* dtheta, double* dout, unsigned flags);

/* Block until everything this context (and the device) was asked to do has
 * finished.  The compute entry points already return drained; this is the
 * explicit fence benchmarks put on both sides of a timed region. */
int plr_synchronize(plr_ctx* ctx);

/* Shape of the resident shard (0,0 before plr_set_data). */
int plr_get_shape(const plr_ctx* ctx, int64_t* n, int64_t* d);

/* Timing of the streaming kernel, measured with HIP events recorded on the
 * context's own stream around the kernel launch only: milliseconds of the
 * last launch and, since the last plr_reset_timing, the sum and the count.
 * Any pointer may be NULL. */
int plr_get_timing(const plr_ctx* ctx, double* last_ms, double* sum_ms,
                   int64_t* launches);
int plr_reset_timing(plr_ctx* ctx);

/* Switch the timing events off (enabled = 0) or back on (the default).  The
 * two event records cost 6-8 us per call (measured: 38.9 -> 33.1 us per
 * plr_loss_grad on a 100 000 x 100 shard), which matters for shards whose
 * pass takes tens of microseconds; with timing off plr_get_timing keeps
 * reporting what it held when it was switched off.  No counterpart in the
 * reference. */
int plr_set_timing(plr_ctx* ctx, int enabled);

/* Tuning and diagnostic switches of a context; no counterpart in the
 * reference.  Keys:
 *   "first_column_is_one"  value != 0: the caller states that column 0 of every
 *        shard it uploads from now on is the constant 1.0 -- the bias column
 *        local_parser prepends (lr.cpp:83).  The library then keeps only the
 *        other d - 1 columns in HBM (a 2^k + 1 wide row streams as a 2^k wide
 *        one), adds theta[0] to every dot product and returns the sum of the
 *        residuals as gsum[0]; every result is what the stored column would
 *        have given.  The upload checks the statement row by row and fails
 *        with PLR_ERR_INVALID at the first row that does not start with 1.0.
 *        Applies from the next plr_set_data / plr_alloc_data.  Default 0.
 *   "column_blocks_two_sweeps"  value != 0: rows wider than 19456 columns are
 *        processed in two sweeps over X (dot products, then updates) instead
 *        of once by cooperating workgroups; applies from the next
 *        plr_set_data / plr_alloc_data.  Default 0.
 *   "team_spin_limit"  how many times a workgroup of the one-read wide-row
 *        pass polls for a partner's partial dot product before it gives up.
 *        Default 4194304; 0 makes every wait give up at once (used to test the
 *        paths below).
 *   "team_fallback"  what happens when such a pass gives up -- its workgroups
 *        must all be resident at once, which other processes or streams on the
 *        device can prevent.  != 0 (default): the pass is run again in two
 *        sweeps, which need no residency, and the caller gets its results; after
 *        two such passes the resident shard stays on two sweeps
 *        (plr_kernel_info says so).  0: the call fails with PLR_ERR_HIP.
 *   "team_lag"  how many rows the rank-1 update of that pass trails the dot
 *        product: 1, 2, or 0 (default) = chosen by the width.  Same results;
 *        applies from the next plr_set_data / plr_alloc_data.
 *   "poll_results"  value != 0 (default): after a pass over rows of up to 1024
 *        stored columns the calling thread watches host memory for the
 *        results, which the last kernel writes there with a pass number behind
 *        them, instead of waiting for the runtime to report the stream
 *        drained (3-4 us sooner).  0: always wait for the stream.  Same
 *        results.
 *   "csv_overlap"  value != 0 (default): plr_set_data_csv parses texts of
 *        256 MiB and more stretch by stretch while the rest is still arriving
 *        from the host, into a shard reserved for an estimated number of rows
 *        (a few rows more than needed stay allocated; when the estimate is too
 *        low the call starts over with 0's way).  0: transfer, count the rows,
 *        reserve exactly that shard, parse.  Same shard contents. */
int plr_set_option(plr_ctx* ctx, const char* key, int64_t value);

/* Read ceiling of this device, measured on the resident shard: a kernel that
 * only streams X (same access pattern as the fused pass, no arithmetic) is
 * launched `reps` times; reports GB/s.  No counterpart in the reference; used
 * by benchmarks to state the fused pass as a fraction of what a pure read
 * sustains. */
int plr_probe_read_bandwidth(plr_ctx* ctx, int reps, double* gb_per_s);

/* Copy ceiling of this device: the runtime's device-to-device copy of `bytes`
 * bytes between two temporary buffers (allocated and freed inside the call),
 * `reps` times after one warm-up; reports GB/s of bytes read plus bytes
 * written.  No counterpart in the reference; benchmarks quote it next to the
 * read ceiling. */
int plr_probe_copy_bandwidth(plr_ctx* ctx, int64_t bytes, int reps, double* gb_per_s);

/* Human-readable description of the kernel variant chosen for the resident
 * shape (tile shape, grid), for logs.  Context-owned, never freed. */
const char* plr_kernel_info(const plr_ctx* ctx);

/* Context-owned message of the last error ("" if none); never freed.
 * plr_last_error(NULL) describes the last failure of a call that takes no
 * context (plr_create, plr_loss_grad_noalloc). */
const char* plr_last_error(const plr_ctx* ctx);

const char* plr_version(void);

#ifdef __cplusplus
}
#endif
#endif /* PLR_H */
