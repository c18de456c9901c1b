// Host-only check of the worker collectives in paralg_lite.hpp (paracel_sync,
// allreduce) with several plain worker processes against one plr_ps_server:
//   plr_comm_check --server_info H:p0,..,p4 --worker_id R --worker_sz W [--rounds K]
// Every round: a barrier, then an all-reduce of (rank + 1) * (round + 1) and of
// an int; between two barriers each worker bumps a shared counter and checks
// after the second one that all W bumps are there (what a barrier is for).
// Prints "ok <rank>" and exits 0, or a message and exits 1.
//   plr_comm_check --hw_queues W
// prints what GPU_MAX_HW_QUEUES reads after limit_hw_queues_of_gpu_sharers(W)
// (or "unset"), for the value found in the environment.
#include <stdlib.h>

#include <iostream>

#include "gpu_turn.hpp"
#include "paralg_lite.hpp"

int main(int argc, char** argv) {
  std::string info;
  int rank = 0, W = 1, rounds = 25;
  for (int i = 1; i + 1 < argc; i += 2) {
    const std::string a = argv[i], v = argv[i + 1];
    if (a == "--server_info") info = v;
    else if (a == "--worker_id") rank = atoi(v.c_str());
    else if (a == "--worker_sz") W = atoi(v.c_str());
    else if (a == "--rounds") rounds = atoi(v.c_str());
    else if (a == "--hw_queues") {
      plr_ps::limit_hw_queues_of_gpu_sharers(atoi(v.c_str()));
      const char* q = getenv("GPU_MAX_HW_QUEUES");
      std::cout << (q ? q : "unset") << std::endl;
      return 0;
    }
  }
  try {
    plr_ps::paralg pa(info, "", 1, rank, W);
    for (int k = 0; k < rounds; ++k) {
      pa.paracel_sync();
      double v = (rank + 1.) * (k + 1.);
      pa.allreduce(v);
      const double want = (k + 1.) * W * (W + 1.) / 2.;
      if (v != want) {
        std::cerr << "round " << k << ": allreduce gave " << v << ", want " << want << std::endl;
        return 1;
      }
      int c = rank + k;
      pa.allreduce(c);
      if (c != W * (W - 1) / 2 + W * k) {
        std::cerr << "round " << k << ": int allreduce gave " << c << std::endl;
        return 1;
      }
      // nobody passes the second barrier before everybody has written
      pa.paracel_write("bump_" + std::to_string(k) + "_" + std::to_string(rank), (double)rank);
      if (k & 1) pa.paracel_sync_arrive();  // every other round: the barrier in two halves
      pa.paracel_sync();
      for (int r = 0; r < W; ++r) {
        const double got =
            pa.paracel_read<double>("bump_" + std::to_string(k) + "_" + std::to_string(r));
        if (got != (double)r) {
          std::cerr << "round " << k << ": worker " << r << "'s write is missing" << std::endl;
          return 1;
        }
      }
    }
    std::cout << "ok " << rank << std::endl;
  } catch (const std::exception& e) {
    std::cerr << e.what() << std::endl;
    return 1;
  }
  return 0;
}
