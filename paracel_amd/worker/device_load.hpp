// paracel_load + local_parser with the parsing done on the device
// (lr.cpp:303-305 and 76-93; ridge.hpp:142-160 is the same parser): the
// worker's share of the text goes to HBM as it lies in the files
// (plr_set_data_csv) and the shard never exists on the host -- except once,
// on its way into the binary cache the next run starts from.
#pragma once

#include <stdlib.h>

#include <chrono>
#include <iostream>
#include <stdexcept>
#include <string>

#include "../../include/plr.h"
#include "shard_io.hpp"

namespace plr_ps {

// True when the shard of worker `rank` of `np` is resident afterwards (n x d,
// d counting the constant first column).  False, with nothing done, when the
// binary cache is fresh (reading it beats any parser), when PLR_HOST_PARSE is
// set, or when the library leaves this input to the host's parser.  The
// parser's errors (a field std::stod rejects, a ragged line) are thrown as
// std::invalid_argument, like parse_lines'.
inline bool load_shard_on_device(plr_ctx* gpu, const std::string& fn, int rank, int np,
                                 int64_t& n, int64_t& d) {
  const char* host = getenv("PLR_HOST_PARSE");
  if (host && *host && *host != '0') return false;
  {
    ShardCacheHeader h;
    FILE* f = nullptr;
    if (open_cache(fn, rank, np, h, f)) {
      fclose(f);
      return false;
    }
  }
  const auto t0 = std::chrono::steady_clock::now();
  OwnedText own;
  owned_text(fn, rank, np, own);
  const int rc = plr_set_data_csv(gpu, own.text.data(), own.len.data(), (int)own.text.size(), ',',
                                  &n, &d);
  if (rc == PLR_ERR_UNSUPPORTED) return false;
  if (rc != PLR_OK) throw std::invalid_argument(plr_last_error(gpu));
  std::cout << "lines got: " << n << std::endl;  // loader.hpp:93
  std::cout << "parsed on the device: " << n << " x " << d << " in "
            << std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count()
            << " s" << std::endl;
  if (n > 0) {
    ParsedShard s;
    s.n = n;
    s.d = d;
    s.X.resize((size_t)n * d);
    s.y.resize(n);
    if (plr_get_data(gpu, 0, n, s.X.data(), d, s.y.data()) != PLR_OK)
      throw std::runtime_error(std::string("plr_get_data: ") + plr_last_error(gpu));
    if (!write_cache(fn, rank, np, s)) std::cout << "shard cache not written" << std::endl;
  }
  return true;
}

}  // namespace plr_ps
