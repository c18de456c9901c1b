// Worker entry point, after the reference's
// alg/classification/logistic_regression/lr_driver.cpp:34-78: the same two
// flags (--server_info, --cfg_file), the same JSON keys (training_input,
// test_input, predict_input, output, update_file, update_func, method, rounds,
// alpha, beta, debug) and the same call order solve -> calc_loss -> test ->
// predict -> dump_result.
//
// A second mode serves the end-to-end benchmark: --synthetic SEED,N,D,SCALE
// builds the shard in memory with the seeded generator instead of parsing a
// file (worker R of W takes rows [N R / W, N (R + 1) / W) of the N-row shard, as
// the loader would hand it its share of a file), runs the rounds against the
// parameter server and prints one JSON line with the end-to-end and GPU-only
// rates; --theta_out writes the final theta as raw doubles (worker 0).
//
// Where the reference takes rank and size from MPI (lr_driver.cpp:36-37, one
// process per worker under mpirun), --worker_id R --worker_sz W name this
// process's place among W plain worker processes that share the server.
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <fstream>
#include <iostream>
#include <map>
#include <sstream>

#include "../datagen/plr_gen.h"
#include "driver_util.hpp"
#include "lr_gpu.hpp"

using plr_ps::logistic_regression_gpu;
using plr_ps::need;
using plr_ps::parse_flat_json;

int main(int argc, char** argv) {
  std::string server_info, cfg_file, synthetic, theta_out, theta0 = "random", update_file,
                                                           update_func = "lr_theta_update";
  int rounds = 100, device = 0, worker_id = 0, worker_sz = 1;
  double alpha = 0.002, beta = 0.1;
  for (int i = 1; i < argc; ++i) {
    std::string a = argv[i], v;
    const size_t eq = a.find('=');
    if (eq != std::string::npos) {
      v = a.substr(eq + 1);
      a = a.substr(0, eq);
    } else if (i + 1 < argc) {
      v = argv[++i];
    }
    if (a == "--server_info") server_info = v;
    else if (a == "--cfg_file") cfg_file = v;
    else if (a == "--synthetic") synthetic = v;
    else if (a == "--theta_out") theta_out = v;
    else if (a == "--theta0") theta0 = v;
    else if (a == "--rounds") rounds = atoi(v.c_str());
    else if (a == "--alpha") alpha = atof(v.c_str());
    else if (a == "--beta") beta = atof(v.c_str());
    else if (a == "--update_file") update_file = v;
    else if (a == "--update_func") update_func = v;
    else if (a == "--device") device = atoi(v.c_str());
    else if (a == "--worker_id") worker_id = atoi(v.c_str());
    else if (a == "--worker_sz") worker_sz = atoi(v.c_str());
    else {
      std::cerr << "[options]\n\t--server_info\n\t--cfg_file\n";
      return 1;
    }
  }
  plr_ps::limit_hw_queues_of_gpu_sharers(worker_sz);  // before the first GPU call
  try {
    if (!synthetic.empty()) {
      unsigned long long seed;
      long long n, d;
      double scale;
      if (sscanf(synthetic.c_str(), "%llx,%lld,%lld,%lf", &seed, &n, &d, &scale) != 4)
        throw std::invalid_argument("--synthetic wants SEEDHEX,N,D,SCALE");
      logistic_regression_gpu lr(server_info, "", "", update_file, update_func, "dgd", rounds,
                                 alpha, beta, false, device, worker_id, worker_sz);
      const long long lo = n * worker_id / worker_sz, hi = n * (worker_id + 1) / worker_sz;
      {
        plr_gen_spec sp = {seed, PLR_GEN_NORMAL, 0, scale, 0.0, 1.0};
        const long long m = hi - lo;
        std::vector<double> X((size_t)m * d), y(m), ts(d);
        plr_gen_X(&sp, lo, m, d, d, X.data(), 16);
        plr_gen_vec(seed, PLR_STREAM_THETA_STAR, PLR_GEN_NORMAL, 1.0, 1.0, d, ts.data());
        plr_gen_labels(&sp, lo, m, d, d, X.data(), ts.data(), y.data(), 16);
        lr.set_samples(X.data(), m, d, d, y.data());
      }
      if (theta0 == "zero") lr.set_theta0(std::vector<double>(d, 0.));
      lr.solve();
      const double loss = lr.calc_loss();
      const double sec = lr.round_seconds(), kms = lr.gpu_kernel_ms();
      if (!theta_out.empty() && worker_id == 0) {
        std::ofstream o(theta_out, std::ios::binary);
        o.write((const char*)lr.get_theta().data(), lr.get_theta().size() * sizeof(double));
      }
      n = hi - lo;  // this worker's rows
      printf("{\"rounds\": %d, \"n\": %lld, \"d\": %lld, \"seconds\": %.6f, "
             "\"iters_per_sec\": %.3f, \"gpu_kernel_ms_per_iter\": %.6f, "
             "\"gpu_only_iters_per_sec\": %.3f, \"final_loss\": %.17g}\n",
             rounds, n, d, sec, rounds / sec, kms / (rounds + 1), 1e3 * (rounds + 1) / kms, loss);
      return 0;
    }
    auto kv = parse_flat_json(cfg_file);
    logistic_regression_gpu lr(server_info, need(kv, "training_input"), need(kv, "output"),
                               need(kv, "update_file"), need(kv, "update_func"),
                               need(kv, "method"), atoi(need(kv, "rounds").c_str()),
                               atof(need(kv, "alpha").c_str()), atof(need(kv, "beta").c_str()),
                               need(kv, "debug") == "true", device, worker_id, worker_sz);
    if (theta0 == "zero")
      lr.set_theta0(std::vector<double>(plr_ps::csv_row_width(need(kv, "training_input")), 0.));
    lr.solve();
    std::cout.precision(17);
    std::cout << "final loss: " << lr.calc_loss() << std::endl;
    if (kv.count("test_input") && !kv["test_input"].empty()) lr.test(kv["test_input"]);
    if (kv.count("predict_input") && !kv["predict_input"].empty()) lr.predict(kv["predict_input"]);
    lr.dump_result();
    if (!theta_out.empty() && worker_id == 0) {
      std::ofstream o(theta_out, std::ios::binary);
      o.write((const char*)lr.get_theta().data(), lr.get_theta().size() * sizeof(double));
    }
  } catch (const std::exception& e) {
    std::cerr << e.what() << std::endl;
    return 1;
  }
  return 0;
}
