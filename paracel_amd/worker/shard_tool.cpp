// Command-line front end of shard_io.hpp (no GPU needed):
//   plr_shard_tool parse <input.csv> <rank> <np>   parse this rank's lines and write the cache
//   plr_shard_tool info  <input.csv> <rank> <np>   validate the cache; print n d
//   plr_shard_tool lines <input.csv> <rank> <np>   print the lines this rank owns
//   plr_shard_tool time  <input.csv> <threads> 0   print n d and the seconds of the line split
//                                                  and of the parse on <threads> threads
//   plr_shard_tool owners <input> <lo_np> <hi_np>  for every np in [lo_np, hi_np] and every rank:
//                                                  "np rank line" per owned line
//   plr_shard_tool selftest <count> <seed> 0       parse_field against std::stod on <count>
//                                                  random field spellings, bit for bit
#include <chrono>
#include <iostream>
#include <random>

#include "shard_io.hpp"

// A random field: mostly decimal spellings around the limits of the fast path
// (digit counts 1..38, exponents around +-22 and +-44, zeros, signs), some spellings
// only std::stod understands, some it rejects.
static std::string random_field(std::mt19937_64& rng) {
  auto pick = [&](int n) { return (int)(rng() % (uint64_t)n); };
  static const char* odd[] = {"inf", "-inf", "nan", "0x1.8p3", " 1.5", "+2.5", "1.5abc", "abc",
                              "-", ".", "e5", "1e", "1e+", "1e400", "1e-400", "4.9e-324", "-0",
                              "0.0", "-0.0e7", "00012.500", "1.", ".5", "-.5e-3", "1E5", "2.5E-7"};
  if (pick(16) == 0) return odd[pick((int)(sizeof odd / sizeof *odd))];
  std::string s;
  if (pick(2)) s += '-';
  const int ni = pick(3) ? pick(12) : pick(20), nf = pick(3) ? pick(12) : pick(20);
  for (int i = 0; i < ni; ++i) s += (char)('0' + (pick(4) == 0 ? 0 : pick(10)));
  if (nf || pick(3) == 0) {
    s += '.';
    for (int i = 0; i < nf; ++i) s += (char)('0' + (pick(4) == 0 ? 0 : pick(10)));
  }
  if (pick(2)) {
    s += pick(2) ? 'e' : 'E';
    const int k = pick(3);
    if (k == 0) s += '-';
    if (k == 1) s += '+';
    s += std::to_string(pick(3) == 0 ? pick(400) : pick(60));
  }
  return s;
}

static int selftest(long count, unsigned long long seed) {
  std::mt19937_64 rng(seed);
  long fast_or_equal = 0, threw = 0;
  for (long i = 0; i < count; ++i) {
    const std::string f = random_field(rng);
    double want = 0., got = 0.;
    bool want_throw = false, got_throw = false;
    try {
      want = std::stod(f);
    } catch (const std::exception&) {
      want_throw = true;
    }
    try {
      got = plr_ps::parse_field(f.data(), f.size());
    } catch (const std::exception&) {
      got_throw = true;
    }
    if (want_throw != got_throw || (!want_throw && memcmp(&want, &got, sizeof want) != 0)) {
      std::cout << "MISMATCH '" << f << "'\n";
      return 1;
    }
    threw += want_throw;
    ++fast_or_equal;
  }
  std::cout << "ok " << fast_or_equal << " fields, " << threw << " rejected by both\n";
  return 0;
}

int main(int argc, char** argv) {
  if (argc == 5 && std::string(argv[1]) == "selftest")
    return selftest(atol(argv[2]), strtoull(argv[3], nullptr, 0));
  if (argc == 5 && std::string(argv[1]) == "owners") {
    try {
      for (int np = atoi(argv[3]); np <= atoi(argv[4]); ++np)
        for (int r = 0; r < np; ++r)
          for (const std::string& l : plr_ps::load_lines(argv[2], r, np))
            std::cout << np << " " << r << " " << l << "\n";
    } catch (const std::exception& e) {
      std::cerr << e.what() << "\n";
      return 1;
    }
    return 0;
  }
  if (argc == 6 && std::string(argv[1]) == "recache") {
    // the fresh cache read through its mapping and written again slab by slab
    // (slabs of argv[5] bytes): the two routes the GPU workers take
    const int rank = atoi(argv[3]), np = atoi(argv[4]);
    plr_ps::MappedShard m;
    if (!plr_ps::map_cache(argv[2], rank, np, m)) {
      std::cout << "stale-or-missing\n";
      return 1;
    }
    const int64_t n = m.n, d = m.d;
    std::vector<double> X(m.X(), m.X() + (size_t)n * d), y(m.y(), m.y() + n);
    const bool ok = plr_ps::write_cache_rows(
        argv[2], rank, np, n, d,
        [&](int64_t r0, int64_t rows, double* Xo, double* yo) {
          memcpy(Xo, X.data() + (size_t)r0 * d, (size_t)rows * d * sizeof(double));
          memcpy(yo, y.data() + r0, (size_t)rows * sizeof(double));
          return true;
        },
        (size_t)atoll(argv[5]));
    std::cout << (ok ? "rewritten " : "failed ") << n << " " << d << "\n";
    return ok ? 0 : 1;
  }
  if (argc != 5) {
    std::cerr << "usage: plr_shard_tool parse|info|lines <input> <rank> <np>\n";
    return 2;
  }
  const std::string cmd = argv[1], input = argv[2];
  const int rank = atoi(argv[3]), np = atoi(argv[4]);
  try {
    if (cmd != "time" && (rank < 0 || np < 1 || rank >= np))
      throw std::invalid_argument("need 0 <= rank < np");
    if (cmd == "lines") {
      for (const std::string& l : plr_ps::load_lines(input, rank, np)) std::cout << l << "\n";
    } else if (cmd == "parse") {
      plr_ps::ParsedShard s = plr_ps::parse_lines(plr_ps::load_lines(input, rank, np));
      if (!plr_ps::write_cache(input, rank, np, s)) throw std::runtime_error("cannot write the cache");
      std::cout << s.n << " " << s.d << "\n";
    } else if (cmd == "time") {
      // the host's loader and parser alone: seconds for the line split and for the
      // parse on <rank> threads (np is ignored: the whole input)
      using clk = std::chrono::steady_clock;
      const auto t0 = clk::now();
      const std::vector<std::string> lines = plr_ps::load_lines(input, 0, 1);
      const auto t1 = clk::now();
      plr_ps::ParsedShard s = plr_ps::parse_lines(lines, ',', rank < 1 ? 1 : rank);
      const auto t2 = clk::now();
      std::cout << s.n << " " << s.d << " " << std::chrono::duration<double>(t1 - t0).count()
                << " " << std::chrono::duration<double>(t2 - t1).count() << "\n";
    } else if (cmd == "info") {
      plr_ps::ParsedShard s;
      if (!plr_ps::read_cache(input, rank, np, s)) {
        std::cout << "stale-or-missing\n";
        return 1;
      }
      std::cout << s.n << " " << s.d << "\n";
    } else {
      throw std::invalid_argument("unknown command " + cmd);
    }
  } catch (const std::exception& e) {
    std::cerr << e.what() << "\n";
    return 1;
  }
  return 0;
}
