// Server-side reducer for the LR model vector: theta_new = theta_old + delta,
// element by element.  Same exported symbol and plugin ABI as the reference's
// alg/classification/logistic_regression/update.cpp:22-34 (lr_theta_update),
// so the worker's cfg keys update_file / update_func keep their meaning.
#include <vector>

#include "ps_plugin.hpp"

extern "C" {
extern plr_ps::update_result lr_theta_update;
// dense twin (see ps_plugin.hpp): the same additions on unpacked doubles
void lr_theta_update_dense(double* theta, const double* delta, size_t n);
}

static std::vector<double> add_delta(std::vector<double> theta, std::vector<double> delta) {
  // the reference walks a.size() entries and reads b[i] for each
  for (size_t i = 0; i < theta.size(); ++i) theta[i] = theta[i] + delta[i];
  return theta;
}

plr_ps::update_result lr_theta_update = plr_ps::update_proxy(add_delta);

void lr_theta_update_dense(double* theta, const double* delta, size_t n) {
  for (size_t i = 0; i < n; ++i) theta[i] = theta[i] + delta[i];
}
