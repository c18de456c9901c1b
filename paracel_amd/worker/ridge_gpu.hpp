// Ridge-regression worker with the shard on the GPU.  Same shape as the
// reference's class ridge_regression (alg/regression/ridge/ridge.hpp:32-195):
// same constructor knobs, the same calls against the parameter server --
//   load -> parse(+bias) -> sync -> write theta0 -> register_bupdate ->
//   { read theta -> delta -> sync -> bupdate -> sync } x rounds -> read theta
// (ridge.hpp:55-101) -- and calc_loss / test / predict / dump_result with the
// reference's formulas and file names (ridge.hpp:103-139), the loops over the
// samples being calls into the C ABI of plr.h.
//
// One deliberate difference, in the trainer: the reference's ipm_learning
// changes theta inside the row loop (theta[i] += t per sample,
// ridge.hpp:78-86) and pushes wgt * (theta - theta_old); rows depend on each
// other there, so it is not a batch pass.  solve() here runs the FULL-BATCH
// form of the same update expression (plr_dgd_delta_linear: every row's t
// evaluated at the theta read at the start of the round, summed), which is to
// ridge what dgd_learning (lr.cpp:109-152) is to logistic regression; the
// workers' deltas add up on the server, so no 1/worker_sz weight is applied.
#pragma once

#include <string>
#include <utility>
#include <vector>

#include "../../include/plr.h"
#include "gpu_turn.hpp"
#include "paralg_lite.hpp"

namespace plr_ps {

class ridge_regression_gpu : public paralg {
 public:
  ridge_regression_gpu(const std::string& hosts_dct_str, const std::string& _input,
                       const std::string& output, const std::string& update_fn,
                       const std::string& update_fcn, int _rounds, double _alpha, double _beta,
                       int device_id = 0, int worker_id = 0, int worker_sz = 1);
  virtual ~ridge_regression_gpu();

  void set_theta0(const std::vector<double>& t0) { theta0 = t0; }

  virtual void solve();         // ridge.hpp:55-61 with the batch trainer
  void batch_learning();        // full-batch rounds (see the note above)
  double calc_loss();           // ridge.hpp:103-113
  void test(const std::string& test_fn);      // ridge.hpp:122-128
  void predict(const std::string& pred_fn);   // ridge.hpp:130-139
  void dump_result();           // ridge.hpp:115-120

  const std::vector<double>& get_theta() const { return theta; }
  const std::vector<double>& get_predictions() const { return pred_z; }

 private:
  void load_and_upload(const std::string& fn);  // paracel_load + local_parser (ridge.hpp:142-160)
  void check(int rc, const char* what);

  std::string input, update_file, update_func;
  int worker_id;
  int rounds;
  double alpha, beta;
  int kdim = 0;
  int64_t n_local = 0, data_dim = 0;
  std::vector<double> theta, theta0;
  std::vector<double> pred_z, pred_samples;
  int64_t pred_dim = 0;
  plr_ctx* gpu = nullptr;
  gpu_turn turn;
};

}  // namespace plr_ps
