// Ridge worker entry point, after the reference's
// alg/regression/ridge/ridge_driver.cpp:29-73: the same two flags
// (--server_info, --cfg_file), the same JSON keys (training_input, test_input,
// predict_input, output, update_file, update_func, rounds, alpha, beta) and
// the same call order solve -> calc_loss -> test -> predict -> dump_result.
// --worker_id / --worker_sz stand in for the MPI rank and size; --theta0 zero
// starts from the zero vector instead of random_double_list; --theta_out
// writes worker 0's final theta as raw doubles.
#include <stdlib.h>

#include <fstream>
#include <iostream>

#include "driver_util.hpp"
#include "ridge_gpu.hpp"

using plr_ps::need;

int main(int argc, char** argv) {
  std::string server_info, cfg_file, theta0 = "random", theta_out;
  int device = 0, worker_id = 0, worker_sz = 1;
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
    else if (a == "--theta0") theta0 = v;
    else if (a == "--theta_out") theta_out = v;
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
    auto kv = plr_ps::parse_flat_json(cfg_file);
    plr_ps::ridge_regression_gpu solver(
        server_info, need(kv, "training_input"), need(kv, "output"), need(kv, "update_file"),
        need(kv, "update_func"), atoi(need(kv, "rounds").c_str()),
        atof(need(kv, "alpha").c_str()), atof(need(kv, "beta").c_str()), device, worker_id,
        worker_sz);
    if (theta0 == "zero")
      solver.set_theta0(
          std::vector<double>(plr_ps::csv_row_width(need(kv, "training_input")), 0.));
    solver.solve();
    std::cout.precision(17);
    std::cout << "final loss: " << solver.calc_loss() << std::endl;
    solver.test(need(kv, "test_input"));
    solver.predict(need(kv, "predict_input"));
    solver.dump_result();
    if (!theta_out.empty() && worker_id == 0) {
      std::ofstream o(theta_out, std::ios::binary);
      o.write((const char*)solver.get_theta().data(), solver.get_theta().size() * sizeof(double));
    }
  } catch (const std::exception& e) {
    std::cerr << e.what() << std::endl;
    return 1;
  }
  return 0;
}
