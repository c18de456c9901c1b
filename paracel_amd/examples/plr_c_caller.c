/* A plain C99 caller of the C ABI in include/plr.h: what a host that is not
 * C++ binds.  Reads a shard and theta from a text file
 *     n d alpha beta
 *     n*d values of X (row-major), n labels, d values of theta
 * makes the shard resident, asks for one round's delta (lr.cpp:125-138) and
 * prints "delta[j] = ..." and the loss sum with 17 significant digits.
 *     plr_c_caller <input.txt> */
#include <stdio.h>
#include <stdlib.h>

#include "plr.h"

static int read_doubles(FILE* f, double* v, long count) {
  long i;
  for (i = 0; i < count; ++i)
    if (fscanf(f, "%lf", &v[i]) != 1) return 0;
  return 1;
}

int main(int argc, char** argv) {
  long n, d, j;
  double alpha, beta, loss = 0.;
  double *X, *y, *theta, *delta;
  plr_ctx* ctx = NULL;
  FILE* f;
  int rc;
  if (argc != 2 || !(f = fopen(argv[1], "r"))) {
    fprintf(stderr, "usage: plr_c_caller <input.txt>\n");
    return 2;
  }
  if (fscanf(f, "%ld %ld %lf %lf", &n, &d, &alpha, &beta) != 4 || n < 0 || d < 1) return 2;
  X = (double*)malloc(sizeof(double) * (size_t)(n * d + 1));
  y = (double*)malloc(sizeof(double) * (size_t)(n + 1));
  theta = (double*)malloc(sizeof(double) * (size_t)d);
  delta = (double*)malloc(sizeof(double) * (size_t)d);
  if (!X || !y || !theta || !delta) return 2;
  if (!read_doubles(f, X, n * d) || !read_doubles(f, y, n) || !read_doubles(f, theta, d)) return 2;
  fclose(f);

  rc = plr_create(&ctx, 0);
  if (rc != PLR_OK) {
    fprintf(stderr, "plr_create: %s\n", plr_last_error(NULL));
    return 1;
  }
  rc = plr_set_data(ctx, X, n, d, d, y);
  if (rc == PLR_OK) rc = plr_dgd_delta(ctx, theta, alpha, beta, delta, &loss);
  if (rc != PLR_OK) {
    fprintf(stderr, "plr: %s\n", plr_last_error(ctx));
    plr_destroy(ctx);
    return 1;
  }
  for (j = 0; j < d; ++j) printf("delta[%ld] = %.17g\n", j, delta[j]);
  printf("loss_sum = %.17g\n", loss);
  printf("%s\n", plr_version());
  plr_destroy(ctx);
  free(X);
  free(y);
  free(theta);
  free(delta);
  return 0;
}
