// Logistic-regression worker with the shard on the GPU.  Same shape as the
// reference's class logistic_regression
// (alg/classification/logistic_regression/lr.hpp:30-81, lr.cpp): same
// constructor knobs, same call order against the parameter server --
//   load -> parse(+bias) -> sync -> write theta0 -> register_bupdate ->
//   { read theta -> delta -> sync -> bupdate -> sync } x rounds -> read theta
// (lr.cpp:301-319,109-152) -- but the three loops over the samples
// (lr.cpp:132-138, 322-330, 361-363) are calls into the C ABI of plr.h.
#pragma once

#include <string>
#include <utility>
#include <vector>

#include "../../include/plr.h"
#include "gpu_turn.hpp"
#include "paralg_lite.hpp"

namespace plr_ps {

class logistic_regression_gpu : public paralg {
 public:
  logistic_regression_gpu(const std::string& hosts_dct_str, const std::string& _input,
                          const std::string& output, const std::string& update_file_name,
                          const std::string& update_func_name, const std::string& method = "dgd",
                          int _rounds = 1, double _alpha = 0.002, double _beta = 0.1,
                          bool _debug = false, int device_id = 0, int worker_id = 0,
                          int worker_sz = 1);
  virtual ~logistic_regression_gpu();

  // lr.cpp:76-93: "f1,...,fk,label" -> [1.0, f1..fk] and label
  void local_parser(const std::vector<std::string>& linelst, char sep = ',');
  // a shard that is already numeric (row-major n x d, no bias column added)
  void set_samples(const double* X, int64_t n, int64_t d, int64_t ldx, const double* y);
  // theta the first round starts from; by default the reference's
  // random_double_list (utils.hpp:116-131: libc random()/RAND_MAX in (0,1))
  void set_theta0(const std::vector<double>& t0) { theta0 = t0; }

  virtual void solve();         // lr.cpp:301-319
  void dgd_learning();          // lr.cpp:109-152
  double calc_loss();           // lr.cpp:321-336
  void test(const std::string& test_fn);        // lr.cpp:348-354
  void predict(const std::string& pred_fn);     // lr.cpp:356-365
  void dump_result();           // lr.cpp:338-346

  const std::vector<double>& get_theta() const { return theta; }
  const std::vector<double>& get_loss_error() const { return loss_error; }
  const std::vector<double>& get_predictions() const { return pred_h; }
  double gpu_kernel_ms() const;  // sum of the streaming-kernel time so far
  double round_seconds() const { return round_sec; }  // wall time inside the rounds loop

 private:
  void load_and_parse(const std::string& fn);  // paracel_load + local_parser, cached
  bool load_on_device(const std::string& fn);  // ... with the text parsed on the device
  void upload();                // flat rows -> HBM, then the host copy is dropped
  void check(int rc, const char* what);

  std::string input, update_file, update_func, learning_method;
  int worker_id;
  int rounds;
  double alpha, beta;
  bool debug;
  int kdim = 0;                 // features without the bias column
  int64_t n_local = 0, data_dim = 0;
  std::vector<double> flat, labels;   // staging only
  std::vector<double> theta, theta0;
  std::vector<double> loss_error;     // debug: n_local entries per round (lr.cpp:139-141)
  std::vector<double> pred_h;
  std::vector<double> pred_samples;   // flattened prediction rows (lr.hpp: pred_samples)
  int64_t pred_dim = 0;
  plr_ctx* gpu = nullptr;
  gpu_turn turn;
  double round_sec = 0.;
};

}  // namespace plr_ps
