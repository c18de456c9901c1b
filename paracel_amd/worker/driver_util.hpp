// What the worker drivers share: the flat JSON configuration file the
// reference's drivers read through json_parser (utils.hpp:133-183) and the
// "--flag value" / "--flag=value" command line.
#pragma once

#include <string.h>

#include <fstream>
#include <map>
#include <sstream>
#include <stdexcept>
#include <string>

namespace plr_ps {

// Flat JSON object of strings, numbers and booleans (what demo_cfg.json holds).
inline std::map<std::string, std::string> parse_flat_json(const std::string& path) {
  std::ifstream f(path);
  if (!f) throw std::invalid_argument("cannot open cfg file " + path);
  std::stringstream ss;
  ss << f.rdbuf();
  const std::string s = ss.str();
  std::map<std::string, std::string> kv;
  size_t i = 0;
  auto skip = [&]() { while (i < s.size() && strchr(" \t\r\n,", s[i])) ++i; };
  auto str = [&]() {
    std::string o;
    ++i;  // opening quote
    while (i < s.size() && s[i] != '"') {
      if (s[i] == '\\' && i + 1 < s.size()) ++i;
      o.push_back(s[i++]);
    }
    ++i;
    return o;
  };
  skip();
  if (i >= s.size() || s[i] != '{') throw std::invalid_argument("cfg: expected '{'");
  ++i;
  for (;;) {
    skip();
    if (i >= s.size()) throw std::invalid_argument("cfg: unterminated object");
    if (s[i] == '}') break;
    if (s[i] != '"') throw std::invalid_argument("cfg: expected a key");
    const std::string key = str();
    skip();
    if (i >= s.size() || s[i] != ':') throw std::invalid_argument("cfg: expected ':'");
    ++i;
    skip();
    if (i >= s.size()) throw std::invalid_argument("cfg: value missing");
    if (s[i] == '"') {
      kv[key] = str();
    } else {
      size_t j = i;
      while (j < s.size() && !strchr(",}\r\n \t", s[j])) ++j;
      kv[key] = s.substr(i, j - i);
      i = j;
    }
  }
  return kv;
}

inline const std::string& need(const std::map<std::string, std::string>& kv, const char* k) {
  auto it = kv.find(k);
  if (it == kv.end()) throw std::invalid_argument(std::string("cfg key missing: ") + k);
  return it->second;
}


// Width of the rows a CSV file yields ("f1,...,fk,label" -> bias + k features).
inline size_t csv_row_width(const std::string& path) {
  std::ifstream f(path);
  std::string first;
  std::getline(f, first);
  size_t k = 0;
  for (char c : first) k += (c == ',');
  return k + 1;
}

}  // namespace plr_ps
