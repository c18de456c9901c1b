#include "ridge_gpu.hpp"

#include "device_load.hpp"

#include <stdlib.h>

#include <iostream>
#include <stdexcept>

namespace plr_ps {

ridge_regression_gpu::ridge_regression_gpu(const std::string& hosts_dct_str,
                                           const std::string& _input, const std::string& output,
                                           const std::string& update_fn,
                                           const std::string& update_fcn, int _rounds,
                                           double _alpha, double _beta, int device_id,
                                           int _worker_id, int _worker_sz)
    : paralg(hosts_dct_str, output, _rounds, _worker_id, _worker_sz),
      input(_input),
      update_file(update_fn),
      update_func(update_fcn),
      worker_id((int)get_worker_id()),
      rounds(_rounds),
      alpha(_alpha),
      beta(_beta),
      turn(device_id, _worker_sz > 1) {
  check(plr_create(&gpu, device_id), "plr_create");
  // every shard this worker uploads starts its rows with the bias 1.0
  // (ridge.hpp:149,168): that column need not be kept in HBM
  check(plr_set_option(gpu, "first_column_is_one", 1), "plr_set_option");
}

ridge_regression_gpu::~ridge_regression_gpu() { plr_destroy(gpu); }

void ridge_regression_gpu::check(int rc, const char* what) {
  if (rc != PLR_OK) throw std::runtime_error(std::string(what) + ": " + plr_last_error(gpu));
}

// "f1,...,fk,target" -> [1.0, f1..fk] and the target: the same line format and
// parser as the logistic worker's (ridge.hpp:142-160 == lr.cpp:76-93), through
// the same binary shard cache
void ridge_regression_gpu::load_and_upload(const std::string& fn) {
  ParsedShard s;
  const int rank = (int)get_worker_id(), np = (int)get_worker_size();
  {
    int64_t n = 0, d = 0;
    // the fresh cache from its mapping, else parsed in HBM (device_load.hpp)
    if (upload_cached_shard(gpu, fn, rank, np, n, d) || load_shard_on_device(gpu, fn, rank, np, n, d)) {
      n_local = n;
      data_dim = d;
      if (kdim == 0 && data_dim > 0) kdim = (int)data_dim - 1;
      return;
    }
  }
  if (!read_cache(fn, rank, np, s)) {
    s = parse_lines(paracel_load(fn));
    if (!write_cache(fn, rank, np, s)) std::cout << "shard cache not written" << std::endl;
  }
  n_local = s.n;
  data_dim = s.d;
  if (kdim == 0 && data_dim > 0) kdim = (int)data_dim - 1;
  check(plr_set_data(gpu, s.X.data(), s.n, s.d, s.d, s.y.data()), "plr_set_data");
}

void ridge_regression_gpu::batch_learning() {
  if (theta0.empty()) {  // random_double_list(data_dim), utils.hpp:116-131
    for (int64_t i = 0; i < data_dim; ++i) {
      double v = random() / static_cast<double>(RAND_MAX);
      while (v == 0 || v == 1.) v = random() / static_cast<double>(RAND_MAX);
      theta0.push_back(v);
    }
  }
  if ((int64_t)theta0.size() != data_dim) throw std::invalid_argument("theta0 has the wrong length");
  theta = theta0;
  paracel_write("theta", theta);
  paracel_register_bupdate(update_file, update_func);
  std::vector<double> delta(data_dim);
  for (int rd = 0; rd < rounds; ++rd) {
    theta = paracel_read<std::vector<double> >("theta");
    paracel_sync_arrive();  // theta is read (see lr_gpu.cpp)
    {
      gpu_turn_guard mine(turn);  // several workers on the GPU: one pass at a time
      check(plr_dgd_delta_linear(gpu, theta.data(), alpha, beta, delta.data(), nullptr),
            "plr_dgd_delta_linear");
    }
    paracel_sync();
    paracel_bupdate("theta", delta);
    paracel_sync();
    std::cout << "worker" << worker_id << " finished round: " << rd << std::endl;
  }
  theta = paracel_read<std::vector<double> >("theta");
}

void ridge_regression_gpu::solve() {
  load_and_upload(input);
  std::cout << "shard on the device: " << plr_kernel_info(gpu) << std::endl;
  paracel_sync();
  batch_learning();
  paracel_sync();
}

double ridge_regression_gpu::calc_loss() {
  double loss = 0.;
  int64_t cnt = 0;
  {
    gpu_turn_guard mine(turn);
    check(plr_calc_loss(gpu, theta.data(), &loss, &cnt, PLR_LOSS_SQUARED), "plr_calc_loss");
  }
  allreduce(loss);  // ridge.hpp:109-112
  int sz = (int)cnt;
  allreduce(sz);
  return loss / static_cast<double>(sz);
}

void ridge_regression_gpu::dump_result() {
  if (worker_id == 0) paracel_dump_vector(theta, "ridge_theta_", "|");
  std::vector<std::pair<std::vector<double>, double> > predv;
  predv.reserve(pred_z.size());
  for (size_t i = 0; i < pred_z.size(); ++i)
    predv.emplace_back(std::vector<double>(pred_samples.begin() + i * pred_dim,
                                           pred_samples.begin() + (i + 1) * pred_dim),
                       pred_z[i]);
  paracel_dump_vector(predv, "pred_v_", "\n");
}

void ridge_regression_gpu::test(const std::string& test_fn) {
  load_and_upload(test_fn);
  std::cout << "loss in test dataset is: " << calc_loss() << std::endl;
  paracel_sync();
}

void ridge_regression_gpu::predict(const std::string& pred_fn) {
  // ridge.hpp:162-174: "f1,...,fk,..." -> [1.0, f1..fk]; no target
  auto lines = paracel_load(pred_fn);
  pred_samples.clear();
  n_local = 0;
  for (const std::string& line : lines) {
    pred_samples.push_back(1.);
    size_t st = 0;
    int got = 0;
    while (got < kdim) {
      const size_t en = line.find(',', st);
      const std::string tok = line.substr(st, en == std::string::npos ? en : en - st);
      if (!tok.empty()) {
        pred_samples.push_back(parse_field(tok.data(), tok.size()));  // std::stod's value and errors
        ++got;
      }
      if (en == std::string::npos) break;
      st = en + 1;
    }
    if (got != kdim) throw std::invalid_argument("predict line has too few fields");
    ++n_local;
  }
  data_dim = pred_dim = kdim + 1;
  const std::vector<double> zeros(n_local, 0.);
  check(plr_set_data(gpu, pred_samples.data(), n_local, data_dim, data_dim, zeros.data()),
        "plr_set_data");
  pred_z.assign(n_local, 0.);
  check(plr_predict_linear(gpu, theta.data(), pred_z.data()), "plr_predict_linear");
  paracel_sync();
}

}  // namespace plr_ps
