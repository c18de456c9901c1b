#include "lr_gpu.hpp"

#include "device_load.hpp"

#include <stdio.h>
#include <stdlib.h>

#include <chrono>
#include <iostream>
#include <stdexcept>

namespace plr_ps {

logistic_regression_gpu::logistic_regression_gpu(
    const std::string& hosts_dct_str, const std::string& _input, const std::string& output,
    const std::string& update_file_name, const std::string& update_func_name,
    const std::string& method, int _rounds, double _alpha, double _beta, bool _debug,
    int device_id, int _worker_id, int _worker_sz)
    : paralg(hosts_dct_str, output, _rounds, _worker_id, _worker_sz),
      input(_input),
      update_file(update_file_name),
      update_func(update_func_name),
      learning_method(method),
      worker_id((int)get_worker_id()),
      rounds(_rounds),
      alpha(_alpha),
      beta(_beta),
      debug(_debug),
      turn(device_id, _worker_sz > 1) {
  check(plr_create(&gpu, device_id), "plr_create");
}

logistic_regression_gpu::~logistic_regression_gpu() { plr_destroy(gpu); }

void logistic_regression_gpu::check(int rc, const char* what) {
  if (rc != PLR_OK)
    throw std::runtime_error(std::string(what) + ": " + plr_last_error(gpu));
}

void logistic_regression_gpu::local_parser(const std::vector<std::string>& linelst, char sep) {
  ParsedShard s = parse_lines(linelst, sep);
  n_local = s.n;
  data_dim = s.d;
  flat.swap(s.X);
  labels.swap(s.y);
  if (kdim == 0 && data_dim > 0) kdim = (int)data_dim - 1;
}

// paracel_load + local_parser, through the binary shard cache when it is fresh
void logistic_regression_gpu::load_and_parse(const std::string& fn) {
  ParsedShard s;
  const int rank = (int)get_worker_id(), np = (int)get_worker_size();
  if (read_cache(fn, rank, np, s)) {
    std::cout << "shard cache hit: " << s.n << " x " << s.d << std::endl;
    n_local = s.n;
    data_dim = s.d;
    flat.swap(s.X);
    labels.swap(s.y);
    if (kdim == 0 && data_dim > 0) kdim = (int)data_dim - 1;
    return;
  }
  local_parser(paracel_load(fn));
  s.n = n_local;
  s.d = data_dim;
  s.X.swap(flat);
  s.y.swap(labels);
  if (!write_cache(fn, rank, np, s)) std::cout << "shard cache not written" << std::endl;
  flat.swap(s.X);
  labels.swap(s.y);
}

// the fresh binary cache sent from its mapping, else paracel_load + local_parser
// on the device (device_load.hpp)
bool logistic_regression_gpu::load_on_device(const std::string& fn) {
  int64_t n = 0, d = 0;
  const int rank = (int)get_worker_id(), np = (int)get_worker_size();
  // the cache's rows start with the bias 1.0 (lr.cpp:83): not kept in HBM
  check(plr_set_option(gpu, "first_column_is_one", 1), "plr_set_option");
  if (!upload_cached_shard(gpu, fn, rank, np, n, d) && !load_shard_on_device(gpu, fn, rank, np, n, d))
    return false;
  n_local = n;
  data_dim = d;
  if (kdim == 0 && data_dim > 0) kdim = (int)data_dim - 1;
  return true;
}

void logistic_regression_gpu::set_samples(const double* X, int64_t n, int64_t d, int64_t ldx,
                                          const double* y) {
  n_local = n;
  data_dim = d;
  check(plr_set_option(gpu, "first_column_is_one", 0), "plr_set_option");  // rows as given
  check(plr_set_data(gpu, X, n, d, ldx, y), "plr_set_data");
  flat.clear();
  labels.clear();
}

void logistic_regression_gpu::upload() {
  // rows built by local_parser / predict start with the bias 1.0 (lr.cpp:83,99):
  // that column need not be kept in HBM
  check(plr_set_option(gpu, "first_column_is_one", 1), "plr_set_option");
  check(plr_set_data(gpu, flat.data(), n_local, data_dim, data_dim, labels.data()),
        "plr_set_data");
  std::vector<double>().swap(flat);
  std::vector<double>().swap(labels);
}

void logistic_regression_gpu::dgd_learning() {
  if (theta0.empty()) {  // random_double_list(data_dim): U(0,1) from libc random()
    for (int64_t i = 0; i < data_dim; ++i) {
      double v = random() / static_cast<double>(RAND_MAX);
      while (v == 0 || v == 1.) v = random() / static_cast<double>(RAND_MAX);
      theta0.push_back(v);
    }
  }
  if ((int64_t)theta0.size() != data_dim) throw std::invalid_argument("theta0 has the wrong length");
  theta = theta0;
  paracel_write("theta", theta);  // first push
  paracel_register_bupdate(update_file, update_func);
  std::vector<double> delta(data_dim);
  using clk = std::chrono::steady_clock;
  // where a round's time goes: read theta, wait for the GPU (other workers' passes),
  // the pass, barrier, bupdate, barrier
  double phase[6] = {0., 0., 0., 0., 0., 0.};
  auto lap = [](clk::time_point& t, double& into) {
    const clk::time_point now = clk::now();
    into += std::chrono::duration<double>(now - t).count();
    t = now;
  };
  const auto t0 = clk::now();
  for (int rd = 0; rd < rounds; ++rd) {
    clk::time_point t = clk::now();
    theta = paracel_read<std::vector<double> >("theta");
    // theta is read: as far as the barrier in front of the bupdate is concerned
    // (nobody updates theta before everybody has read it) this worker has arrived
    if (!debug) paracel_sync_arrive();
    lap(t, phase[0]);
    // lr.cpp:125-142 in one fused pass over the resident shard.  With debug the
    // reference pushes calc_loss() after EVERY sample (lr.cpp:139-141) -- theta
    // does not change inside the round, so these are n_local copies of the
    // global mean loss at the theta just read, which is what is recorded here
    // (one fused pass and the two all-reduces of lr.cpp:331-335 per round
    // instead of n_local passes)
    double loss_sum = 0.;
    {
      gpu_turn_guard mine(turn);  // several workers on the GPU: one pass at a time
      lap(t, phase[1]);
      check(plr_dgd_delta(gpu, theta.data(), alpha, beta, delta.data(),
                          debug ? &loss_sum : nullptr),
            "plr_dgd_delta");
      lap(t, phase[2]);
    }
    if (debug) {
      double total = loss_sum;
      int cnt = (int)n_local;
      allreduce(total);
      allreduce(cnt);
      loss_error.insert(loss_error.end(), (size_t)n_local, cnt ? total / (double)cnt : 0.);
    }
    paracel_sync();
    lap(t, phase[3]);
    paracel_bupdate("theta", delta);
    lap(t, phase[4]);
    paracel_sync();
    lap(t, phase[5]);
    std::cout << "worker" << get_worker_id() << " finished round: " << rd << std::endl;
  }
  round_sec += std::chrono::duration<double>(clk::now() - t0).count();
  if (rounds > 0) {
    char line[256];
    const double ms = 1e3 / rounds;
    snprintf(line, sizeof line,
             "worker%d ms per round: read theta %.3f, wait for the GPU %.3f, pass %.3f, "
             "barrier %.3f, bupdate %.3f, barrier %.3f",
             (int)get_worker_id(), phase[0] * ms, phase[1] * ms, phase[2] * ms, phase[3] * ms,
             phase[4] * ms, phase[5] * ms);
    std::cout << line << std::endl;
  }
  theta = paracel_read<std::vector<double> >("theta");  // last pull
}

void logistic_regression_gpu::solve() {
  if (!input.empty() && !load_on_device(input)) {
    load_and_parse(input);
    upload();
  }
  std::cout << "shard on the device: " << plr_kernel_info(gpu) << std::endl;
  paracel_sync();
  if (learning_method == "dgd") {
    dgd_learning();
  } else {
    // ipm/downpour/agd update theta inside the row loop (lr.cpp:179-182,...):
    // a serial dependence between rows, not a batch gradient
    std::cerr << "method do not support" << std::endl;
  }
  paracel_sync();
}

double logistic_regression_gpu::calc_loss() {
  double loss = 0.;
  int64_t cnt = 0;
  {
    gpu_turn_guard mine(turn);
    check(plr_calc_loss(gpu, theta.data(), &loss, &cnt, PLR_LOSS_REFERENCE), "plr_calc_loss");
  }
  allreduce(loss);  // lr.cpp:331-334
  int sz = (int)cnt;
  allreduce(sz);
  return loss / static_cast<double>(sz);
}

void logistic_regression_gpu::dump_result() {
  if (worker_id == 0) {
    paracel_dump_vector(theta, "lr_theta_", "|");
    if (debug) paracel_dump_vector(loss_error, "lr_loss_error_", "\n");
  }
  // lr.cpp:346: (sample, h) pairs, one "x0,...,xk:h" line each (ps.hpp:1312-1319)
  if (!pred_h.empty()) {
    std::vector<std::pair<std::vector<double>, double> > predv;
    predv.reserve(pred_h.size());
    for (size_t i = 0; i < pred_h.size(); ++i)
      predv.emplace_back(std::vector<double>(pred_samples.begin() + i * pred_dim,
                                             pred_samples.begin() + (i + 1) * pred_dim),
                         pred_h[i]);
    paracel_dump_vector(predv, "pred_v_", "\n");
  }
}

void logistic_regression_gpu::test(const std::string& test_fn) {
  if (!load_on_device(test_fn)) {
    load_and_parse(test_fn);
    upload();
  }
  std::cout << "loss in test dataset is: " << calc_loss() << std::endl;
  paracel_sync();
}

void logistic_regression_gpu::predict(const std::string& pred_fn) {
  // lr.cpp:95-107: "f1,...,fk,..." -> [1.0, f1..fk]; no label
  auto lines = paracel_load(pred_fn);
  flat.clear();
  labels.clear();
  n_local = 0;
  for (const std::string& line : lines) {
    flat.push_back(1.);
    size_t st = 0;
    int got = 0;
    while (got < kdim) {
      const size_t en = line.find(',', st);
      const std::string tok = line.substr(st, en == std::string::npos ? en : en - st);
      if (!tok.empty()) {
        flat.push_back(parse_field(tok.data(), tok.size()));  // std::stod's value and errors
        ++got;
      }
      if (en == std::string::npos) break;
      st = en + 1;
    }
    if (got != kdim) throw std::invalid_argument("predict line has too few fields");
    labels.push_back(0.);
    ++n_local;
  }
  data_dim = kdim + 1;
  pred_samples = flat;  // kept for dump_result, as the reference keeps pred_samples
  pred_dim = data_dim;
  upload();
  pred_h.assign(n_local, 0.);
  check(plr_predict(gpu, theta.data(), pred_h.data()), "plr_predict");
  paracel_sync();
}

double logistic_regression_gpu::gpu_kernel_ms() const {
  double sum = 0.;
  plr_get_timing(gpu, nullptr, &sum, nullptr);
  return sum;
}

}  // namespace plr_ps
