// Command-line front end of shard_io.hpp (no GPU needed):
//   plr_shard_tool parse <input.csv> <rank> <np>   parse this rank's lines and write the cache
//   plr_shard_tool info  <input.csv> <rank> <np>   validate the cache; print n d
//   plr_shard_tool lines <input.csv> <rank> <np>   print the lines this rank owns
#include <iostream>

#include "shard_io.hpp"

int main(int argc, char** argv) {
  if (argc != 5) {
    std::cerr << "usage: plr_shard_tool parse|info|lines <input> <rank> <np>\n";
    return 2;
  }
  const std::string cmd = argv[1], input = argv[2];
  const int rank = atoi(argv[3]), np = atoi(argv[4]);
  try {
    if (rank < 0 || np < 1 || rank >= np) throw std::invalid_argument("need 0 <= rank < np");
    if (cmd == "lines") {
      for (const std::string& l : plr_ps::load_lines(input, rank, np)) std::cout << l << "\n";
    } else if (cmd == "parse") {
      plr_ps::ParsedShard s = plr_ps::parse_lines(plr_ps::load_lines(input, rank, np));
      if (!plr_ps::write_cache(input, rank, np, s)) throw std::runtime_error("cannot write the cache");
      std::cout << s.n << " " << s.d << "\n";
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
