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
  const auto t1 = std::chrono::steady_clock::now();
  std::cout << "lines got: " << n << std::endl;  // loader.hpp:93
  std::cout << "parsed on the device: " << n << " x " << d << " in "
            << std::chrono::duration<double>(t1 - t0).count() << " s" << std::endl;
  if (n > 0) {
    // into the cache slab by slab: the shard is never whole in host memory
    const bool ok = write_cache_rows(fn, rank, np, n, d,
                                     [&](int64_t r0, int64_t m, double* X, double* y) {
                                       return plr_get_data(gpu, r0, m, X, d, y) == PLR_OK;
                                     });
    if (!ok) std::cout << "shard cache not written" << std::endl;
    else
      std::cout << "shard cache written in "
                << std::chrono::duration<double>(std::chrono::steady_clock::now() - t1).count()
                << " s" << std::endl;
  }
  return true;
}

// The fresh binary cache sent to the device from its mapping (no copy of the
// shard in the process).  False, with nothing done, when there is no fresh
// cache.  The rows start with the constant 1.0 local_parser prepends; the
// caller has told the library so (option "first_column_is_one") or not.
inline bool upload_cached_shard(plr_ctx* gpu, const std::string& fn, int rank, int np, int64_t& n,
                                int64_t& d) {
  const auto t0 = std::chrono::steady_clock::now();
  MappedShard m;
  if (!map_cache(fn, rank, np, m)) return false;
  if (plr_set_data(gpu, m.X(), m.n, m.d, m.d, m.y()) != PLR_OK)
    throw std::runtime_error(std::string("plr_set_data: ") + plr_last_error(gpu));
  n = m.n;
  d = m.d;
  std::cout << "shard cache hit: " << n << " x " << d << ", on the device in "
            << std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count()
            << " s" << std::endl;
  return true;
}

}  // namespace plr_ps
