// Turn-taking of several worker processes at one GPU.
#pragma once

#include <fcntl.h>
#include <stdlib.h>
#include <sys/file.h>
#include <unistd.h>

#include <stdexcept>
#include <string>

namespace plr_ps {

// Several worker processes on one GPU take turns at it.  Passes of different
// processes that run side by side do not add up: each is a persistent grid
// sized to the whole device, and the device shares itself out between
// processes in coarse slices (measured on 2 M x 512 rows: two workers' halves
// 0.89 ms each instead of 0.58).  An advisory lock on a per-device
// file (flock: released by the kernel when its holder dies) makes a pass
// exclusive among the workers of this box; it also gives the one-read pass over
// rows wider than 19456 columns the residency it needs (should another
// process hold compute units all the same, that pass gives up and runs again
// in two sweeps inside the library).  With one worker the lock is never taken.
class gpu_turn {
 public:
  gpu_turn(int device, bool shared) {
    if (!shared) return;
    const std::string path =
        "/tmp/plr_gpu_turn." + std::to_string((long)getuid()) + "." + std::to_string(device);
    fd_ = open(path.c_str(), O_CREAT | O_RDWR | O_CLOEXEC, 0600);
    if (fd_ < 0) throw std::runtime_error("cannot open " + path);
  }
  ~gpu_turn() {
    if (fd_ >= 0) close(fd_);
  }
  gpu_turn(const gpu_turn&) = delete;
  gpu_turn& operator=(const gpu_turn&) = delete;
  void lock() {
    if (fd_ < 0) return;
    while (flock(fd_, LOCK_EX) != 0) {
    }
  }
  void unlock() {
    if (fd_ >= 0) flock(fd_, LOCK_UN);
  }

 private:
  int fd_ = -1;
};

// To be called before the process's first GPU call when worker_sz > 1 workers
// share the GPU.  The runtime spreads a process's streams (the pass's and the
// eight upload lanes') over up to 4 hardware queues; the device serves 16 such
// queues side by side, and with more in existence -- measured: four workers
// and one idle process that had used the GPU before, 20 queues -- it
// multiplexes them, and every pass, although it runs alone, takes 2.7 times as
// long (0.79 ms instead of 0.29 on 500 000 x 512 rows; 220 rounds a second
// instead of 600).  Two queues per worker (one from 8 workers on) keep the
// total below that; the upload loses nothing measurable.  A smaller value
// already in the environment is left alone, a larger one (4 is the runtime's
// default) is lowered.
inline void limit_hw_queues_of_gpu_sharers(int worker_sz) {
  if (worker_sz <= 1) return;
  const int want = worker_sz > 7 ? 1 : 2;
  const char* cur = getenv("GPU_MAX_HW_QUEUES");
  if (cur && atoi(cur) >= 1 && atoi(cur) <= want) return;
  setenv("GPU_MAX_HW_QUEUES", want == 1 ? "1" : "2", /*overwrite=*/1);
}

struct gpu_turn_guard {
  explicit gpu_turn_guard(gpu_turn& t) : t_(t) { t_.lock(); }
  ~gpu_turn_guard() { t_.unlock(); }
  gpu_turn& t_;
};

}  // namespace plr_ps
