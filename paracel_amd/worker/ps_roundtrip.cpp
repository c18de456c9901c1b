// Round-trip timing of the two parameter-server calls a DGD round makes --
// paracel_read("theta") and paracel_bupdate("theta", delta) -- through the
// worker-side client against a running plr_ps_server, without a GPU: what a
// round costs besides the gradient (reference lr.cpp:129,143-145).
//
// Usage: plr_ps_roundtrip --server_info HOST:p0,..,p4 --update_file liblr_update.so
//                         [--update_func lr_theta_update] [--d 512,1001,16385]
//                         [--iters 2000] [--warmup 200]
// Prints one JSON line per width: microseconds per call and an FNV-1a hash
// of the final theta's bytes (theta0_i = 0.25 + i/2^20, delta_i =
// ((i mod 7) - 3)/1024, added warmup + iters times), so that a caller can
// check the value that came back against plain additions.
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "paralg_lite.hpp"

using namespace plr_ps;

static uint64_t fnv1a(const void* p, size_t n) {
  const unsigned char* b = (const unsigned char*)p;
  uint64_t h = 1469598103934665603ull;
  for (size_t i = 0; i < n; ++i) h = (h ^ b[i]) * 1099511628211ull;
  return h;
}

int main(int argc, char** argv) {
  std::string info, file, func = "lr_theta_update", widths = "512,1001,16385";
  int iters = 2000, warmup = 200;
  for (int i = 1; i + 1 < argc; i += 2) {
    const std::string a = argv[i], v = argv[i + 1];
    if (a == "--server_info") info = v;
    else if (a == "--update_file") file = v;
    else if (a == "--update_func") func = v;
    else if (a == "--d") widths = v;
    else if (a == "--iters") iters = atoi(v.c_str());
    else if (a == "--warmup") warmup = atoi(v.c_str());
    else {
      fprintf(stderr, "unknown option %s\n", a.c_str());
      return 2;
    }
  }
  if (info.empty() || file.empty()) {
    fprintf(stderr, "need --server_info and --update_file\n");
    return 2;
  }
  try {
    paralg pa(info);
    if (!pa.paracel_register_bupdate(file, func)) {
      fprintf(stderr, "register_bupdate failed\n");
      return 1;
    }
    size_t st = 0;
    while (st < widths.size()) {
      size_t en = widths.find(',', st);
      if (en == std::string::npos) en = widths.size();
      const int d = atoi(widths.substr(st, en - st).c_str());
      st = en + 1;
      if (d < 1) continue;
      const std::string key = "theta_" + std::to_string(d);
      std::vector<double> theta(d), delta(d);
      for (int i = 0; i < d; ++i) {
        theta[i] = 0.25 + i / 1048576.0;
        delta[i] = ((i % 7) - 3) / 1024.0;
      }
      pa.paracel_write(key, theta);
      double t_read = 0., t_upd = 0.;
      for (int r = 0; r < warmup + iters; ++r) {
        const auto t0 = std::chrono::steady_clock::now();
        theta = pa.paracel_read<std::vector<double> >(key);
        const auto t1 = std::chrono::steady_clock::now();
        pa.paracel_bupdate(key, delta);
        const auto t2 = std::chrono::steady_clock::now();
        if (r >= warmup) {
          t_read += std::chrono::duration<double, std::micro>(t1 - t0).count();
          t_upd += std::chrono::duration<double, std::micro>(t2 - t1).count();
        }
      }
      theta = pa.paracel_read<std::vector<double> >(key);
      printf("{\"d\": %d, \"iters\": %d, \"read_us\": %.2f, \"bupdate_us\": %.2f, "
             "\"theta_fnv1a\": \"%016llx\"}\n",
             d, iters, t_read / iters, t_upd / iters,
             (unsigned long long)fnv1a(theta.data(), theta.size() * sizeof(double)));
      fflush(stdout);
    }
  } catch (const std::exception& e) {
    fprintf(stderr, "plr_ps_roundtrip: %s\n", e.what());
    return 1;
  }
  return 0;
}
