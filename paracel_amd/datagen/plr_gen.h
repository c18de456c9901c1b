/* Seeded synthetic-shard generator (host only); see plr_gen.c. */
#ifndef PLR_GEN_H
#define PLR_GEN_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

enum { PLR_GEN_NORMAL = 0, PLR_GEN_UNIFORM = 1 };
enum { PLR_STREAM_X = 1, PLR_STREAM_ZERO = 2, PLR_STREAM_OUTLIER = 3,
       PLR_STREAM_LABEL = 4, PLR_STREAM_THETA = 5, PLR_STREAM_THETA_STAR = 6 };

typedef struct {
  uint64_t seed;
  int32_t kind;          /* PLR_GEN_NORMAL: scale*N(0,1); PLR_GEN_UNIFORM: U[-scale,scale] */
  int32_t outlier_mod;   /* >0: rows whose key % outlier_mod == 0 are scaled */
  double scale;
  double zero_prob;      /* each entry is exactly 0 with this probability */
  double outlier_scale;
} plr_gen_spec;

/* rows [row0, row0+nrows) of the shard into X (row-major, pitch ldx >= d;
 * pad columns are zeroed).  Any split into row ranges gives the same bytes. */
void plr_gen_X(const plr_gen_spec* sp, int64_t row0, int64_t nrows, int64_t d,
               int64_t ldx, double* X, int threads);
/* a length-n vector (theta, theta*); entries kept with prob nonzero_frac. */
void plr_gen_vec(uint64_t seed, uint64_t stream, int kind, double scale,
                 double nonzero_frac, int64_t n, double* out);
/* y_i = 1.0 if u_i < sigmoid(x_i . theta_star) else 0.0 */
void plr_gen_labels(const plr_gen_spec* sp, int64_t row0, int64_t nrows,
                    int64_t d, int64_t ldx, const double* X,
                    const double* theta_star, double* y, int threads);
double plr_gen_u01(uint64_t seed, uint64_t stream, uint64_t i, uint64_t j);
double plr_gen_normal(uint64_t seed, uint64_t stream, uint64_t i, uint64_t j);

#ifdef __cplusplus
}
#endif
#endif
