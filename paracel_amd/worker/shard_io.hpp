// Host-side producer of the shard the GPU keeps: file -> this worker's lines
// -> numeric rows, plus a binary cache of the parsed shard so that the text
// is parsed once (std::stod over ~20 GB of text per 8 GB of doubles is the
// real end-to-end cost of a file-fed run).
//
//   expand_input: a file, a directory (every file below it) or a glob pattern
//                (include/utils/ext_utility.hpp:113-160).
//   load_lines : the reference's "linesplit" rule -- the files are laid end
//                to end, cut into np equal byte ranges, the last one running
//                to the end; a range owns the lines that START inside it
//                (include/load/partition.hpp:57-86,121-175, reached from
//                paralg::paracel_load, include/ps.hpp:178-197).
//   parse_lines: logistic_regression::local_parser (lr.cpp:76-93):
//                "f1,...,fk,label" -> [1.0, f1..fk] and the label; empty
//                fields are dropped as str_split does
//                (include/utils/ext_utility.hpp:38-50); std::stod semantics.
//                Lines are parsed by several threads; the result does not
//                depend on the thread count.
//   *_cache    : "<input>.plrshard.<rank>of<np>": header + X (row-major,
//                n x d doubles, bias column included) + y.  Rejected unless
//                magic, version, input size and input mtime all match.
#pragma once

#include <fcntl.h>
#include <glob.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <stdexcept>
#include <memory>
#include <string>
#include <thread>
#include <vector>

namespace plr_ps {

inline bool is_regular_file(const std::string& f) {
  struct stat st;
  return stat(f.c_str(), &st) == 0 && S_ISREG(st.st_mode);
}
inline bool is_directory(const std::string& f) {
  struct stat st;
  return stat(f.c_str(), &st) == 0 && S_ISDIR(st.st_mode);
}

inline std::vector<std::string> glob_paths(const std::string& pattern) {
  glob_t g;
  std::vector<std::string> out;
  if (glob(pattern.c_str(), GLOB_TILDE, nullptr, &g) == 0)
    for (size_t i = 0; i < g.gl_pathc; ++i) out.push_back(g.gl_pathv[i]);
  globfree(&g);
  return out;
}

inline void expand_dir(const std::string& dir, std::vector<std::string>& out) {
  const std::string base = (!dir.empty() && dir.back() == '/') ? dir : dir + "/";
  for (const std::string& name : glob_paths(base + "*")) {
    if (is_regular_file(name)) out.push_back(name);
    else if (is_directory(name)) expand_dir(name, out);
  }
}

// 'demo.txt' | 'demo_dir' | 'demo_dir/*.csv'
inline std::vector<std::string> expand_input(const std::string& name) {
  std::vector<std::string> out;
  if (is_regular_file(name)) out.push_back(name);
  else if (is_directory(name)) expand_dir(name, out);
  else out = glob_paths(name);
  return out;
}

// One input file's place in the byte stream formed by all inputs end to end.
struct FileSpan {
  std::string path;
  int64_t begin = 0, end = 0;  // [begin, end) in the stream
};

inline std::vector<FileSpan> stream_layout(const std::vector<std::string>& files) {
  std::vector<FileSpan> spans;
  int64_t pos = 0;
  for (const std::string& f : files) {
    struct stat st;
    if (stat(f.c_str(), &st) != 0 || !S_ISREG(st.st_mode))
      throw std::runtime_error("cannot open " + f);
    FileSpan s;
    s.path = f;
    s.begin = pos;
    s.end = pos += (int64_t)st.st_size;
    spans.push_back(s);
  }
  return spans;
}

// Byte range of the stream that worker `rank` of `np` owns: np equal parts of
// floor(total / np) bytes, the last one taking the remainder
// (include/load/partition.hpp:57-86 with one block per worker).
inline void owned_range(int64_t total, int rank, int np, int64_t& lo, int64_t& hi) {
  const int64_t part = total / np;
  lo = (int64_t)rank * part;
  hi = (rank == np - 1) ? total : lo + part;
}

// A read-only mapping of one file, released on scope exit.
class MappedFile {
 public:
  explicit MappedFile(const std::string& path, int64_t size) : size_(size) {
    if (size_ == 0) return;
    const int fd = open(path.c_str(), O_RDONLY);
    if (fd < 0) throw std::runtime_error("cannot open " + path);
    void* p = mmap(nullptr, (size_t)size_, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (p == MAP_FAILED) throw std::runtime_error("cannot map " + path);
    data_ = static_cast<const char*>(p);
  }
  ~MappedFile() {
    if (data_) munmap(const_cast<char*>(data_), (size_t)size_);
  }
  MappedFile(const MappedFile&) = delete;
  MappedFile& operator=(const MappedFile&) = delete;
  const char* data() const { return data_; }

 private:
  const char* data_ = nullptr;
  int64_t size_;
};

// The lines of one file whose first byte lies in [lo, hi) (file offsets).  A
// line starts at offset 0 or right after a newline, and runs to the next
// newline or the end of the file; the one that starts before hi is taken
// whole even when it runs past hi.  Blank lines are dropped.
inline void lines_starting_in(const char* text, int64_t size, int64_t lo, int64_t hi,
                              std::vector<std::string>& out) {
  if (lo < 0) lo = 0;
  if (hi > size) hi = size;
  int64_t pos = lo;
  if (pos > 0 && text[pos - 1] != '\n') {  // inside a line that belongs to an earlier range
    const void* nl = memchr(text + pos, '\n', (size_t)(size - pos));
    if (!nl) return;
    pos = static_cast<const char*>(nl) - text + 1;
  }
  while (pos < hi) {
    const void* nl = memchr(text + pos, '\n', (size_t)(size - pos));
    const int64_t stop = nl ? static_cast<const char*>(nl) - text : size;
    if (stop > pos) out.emplace_back(text + pos, (size_t)(stop - pos));
    pos = stop + 1;
  }
}

// The reference's "linesplit" load (paralg::paracel_load, include/ps.hpp:178-197
// -> loader::fixload, include/load/loader.hpp:81-96 -> partition.hpp:121-175):
// worker `rank` gets the lines that start inside its byte range of the stream.
// Every line of the input goes to exactly one worker, in stream order.  (On
// input with blank lines the reference stops reading a file at the first one
// when its range runs on into the next file, and hands them to the parser
// otherwise; here they are skipped.)
inline std::vector<std::string> load_lines(const std::string& input, int rank, int np) {
  if (np < 1 || rank < 0 || rank >= np) throw std::invalid_argument("bad worker rank");
  const std::vector<std::string> files = expand_input(input);
  if (files.empty()) throw std::runtime_error("cannot open " + input);
  const std::vector<FileSpan> spans = stream_layout(files);
  int64_t lo = 0, hi = 0;
  owned_range(spans.back().end, rank, np, lo, hi);
  std::vector<std::string> lines;
  for (const FileSpan& f : spans) {
    if (f.end <= lo || f.begin >= hi || f.end == f.begin) continue;  // no byte of it is ours
    const MappedFile m(f.path, f.end - f.begin);
    lines_starting_in(m.data(), f.end - f.begin, lo - f.begin, hi - f.begin, lines);
  }
  return lines;
}

// The same share of the input as load_lines returns, as it lies in the files:
// per file one stretch of text holding exactly the lines that start inside the
// worker's byte range (for a parser that takes the text itself).  The
// mappings live as long as the object.
struct OwnedText {
  std::vector<std::unique_ptr<MappedFile> > files;
  std::vector<const char*> text;
  std::vector<int64_t> len;
};

inline void owned_text(const std::string& input, int rank, int np, OwnedText& out) {
  if (np < 1 || rank < 0 || rank >= np) throw std::invalid_argument("bad worker rank");
  const std::vector<std::string> files = expand_input(input);
  if (files.empty()) throw std::runtime_error("cannot open " + input);
  const std::vector<FileSpan> spans = stream_layout(files);
  int64_t lo = 0, hi = 0;
  owned_range(spans.back().end, rank, np, lo, hi);
  for (const FileSpan& f : spans) {
    if (f.end <= lo || f.begin >= hi || f.end == f.begin) continue;  // no byte of it is ours
    const int64_t size = f.end - f.begin;
    std::unique_ptr<MappedFile> m(new MappedFile(f.path, size));
    const char* t = m->data();
    int64_t b = lo - f.begin < 0 ? 0 : lo - f.begin;
    int64_t e = hi - f.begin > size ? size : hi - f.begin;
    if (b > 0 && t[b - 1] != '\n') {  // inside a line that belongs to an earlier range
      const void* nl = memchr(t + b, '\n', (size_t)(size - b));
      if (!nl) continue;
      b = static_cast<const char*>(nl) - t + 1;
    }
    if (b >= e) continue;  // no line starts inside the range
    if (t[e - 1] != '\n') {  // the line that holds the range's last byte is taken whole
      const void* nl = memchr(t + e, '\n', (size_t)(size - e));
      e = nl ? static_cast<const char*>(nl) - t + 1 : size;
    }
    out.text.push_back(t + b);
    out.len.push_back(e - b);
    out.files.push_back(std::move(m));
  }
}

struct ParsedShard {
  int64_t n = 0, d = 0;          // d counts the bias column
  std::vector<double> X, y;      // X: n x d row-major
};

// m * 10^e for 1 <= m < 2^64 and |e| <= 44, correctly rounded -- or false when
// 106 bits cannot tell on which side of a rounding boundary the value lies.
// The integer is split exactly into two doubles and scaled in double-double
// arithmetic: the quotient (product) of the high part, its exact remainder
// (error) by FMA, the correction from the low part; the result is good to
// about 2^-100, and the high word is taken only when the low word is not within
// 2^-30 of a unit in the last place of the midpoint towards the neighbour on
// its side (exact ties included).  Every operation below must stay a single
// IEEE operation: this file is compiled with -ffp-contract=off.  The device
// parser (csrc/plr_csv.hpp) runs the same sequence.
inline bool scale_exact_dd(uint64_t m, int e, const double* pow10, double& out) {
  double h = (double)m;
  double l = (double)(int64_t)(m - (uint64_t)h);
  int left = e < 0 ? -e : e;
  while (left > 0) {
    const int k = left > 22 ? 22 : left;
    const double p = pow10[k];
    left -= k;
    double a, b;
    if (e < 0) {
      a = h / p;
      const double r = std::fma(-a, p, h) + l;
      b = r / p;
    } else {
      a = h * p;
      b = std::fma(h, p, -a) + l * p;
    }
    h = a + b;
    l = b + (a - h);
  }
  int64_t hb;
  memcpy(&hb, &h, sizeof hb);
  hb += l < 0. ? -1 : 1;
  double nb;
  memcpy(&nb, &hb, sizeof nb);
  const double half = 0.5 * std::fabs(nb - h);
  if (std::fabs(std::fabs(l) - half) <= half * 9.313225746154785e-10) return false;  // 2^-30
  out = h;
  return true;
}

// std::stod's value for one field, without the library call for the common
// spellings [-]digits[.digits][e[+-]digits]:
//   * at most 15 significant digits and a decimal exponent within +-22: the
//     digits are an exact double, 10^|e| is an exact double, and the one
//     multiplication or division rounds once -- the correctly rounded result,
//     which is what strtod returns (Clinger's fast path);
//   * up to 19 significant digits and an exponent within +-44: scale_exact_dd.
// Every other spelling (more digits, hex floats, inf, nan, leading blanks or
// '+', trailing garbage) and every error goes through std::stod itself, so the
// exceptions are the reference's too.
inline double parse_field(const char* p, size_t len) {
  static const double kPow10[23] = {1e0,  1e1,  1e2,  1e3,  1e4,  1e5,  1e6,  1e7,
                                    1e8,  1e9,  1e10, 1e11, 1e12, 1e13, 1e14, 1e15,
                                    1e16, 1e17, 1e18, 1e19, 1e20, 1e21, 1e22};
  const char* q = p;
  const char* const end = p + len;
  bool neg = false;
  if (q < end && *q == '-') {
    neg = true;
    ++q;
  }
  uint64_t m = 0;
  int sig = 0, ndig = 0, frac = 0;
  for (; q < end && *q >= '0' && *q <= '9'; ++q, ++ndig) {
    m = m * 10 + (uint64_t)(*q - '0');
    if (m) ++sig;
    if (sig > 19) goto slow;
  }
  if (q < end && *q == '.') {
    ++q;
    for (; q < end && *q >= '0' && *q <= '9'; ++q, ++ndig, ++frac) {
      m = m * 10 + (uint64_t)(*q - '0');
      if (m) ++sig;
      if (sig > 19) goto slow;
    }
  }
  if (ndig == 0) goto slow;
  {
    int e10 = 0;
    if (q < end && (*q == 'e' || *q == 'E')) {
      ++q;
      bool eneg = false;
      if (q < end && (*q == '+' || *q == '-')) eneg = (*q++ == '-');
      int ed = 0;
      for (; q < end && *q >= '0' && *q <= '9'; ++q, ++ed) {
        e10 = e10 * 10 + (*q - '0');
        if (e10 > 9999) goto slow;
      }
      if (ed == 0) goto slow;
      if (eneg) e10 = -e10;
    }
    if (q != end) goto slow;
    e10 -= frac;
    if (e10 < -44 || e10 > 44) goto slow;
    double v = 0.;
    if (sig <= 15 && e10 >= -22 && e10 <= 22) {
      v = (double)m;
      v = (e10 < 0) ? v / kPow10[-e10] : v * kPow10[e10];
    } else if (m != 0 && !scale_exact_dd(m, e10, kPow10, v)) {
      goto slow;
    }
    return neg ? -v : v;
  }
slow:
  return std::stod(std::string(p, len));  // throws like the reference
}

inline void parse_one_line(const std::string& line, char sep, std::vector<double>& fields) {
  fields.clear();
  size_t st = 0;
  for (;;) {
    const size_t en = line.find(sep, st);
    const size_t len = (en == std::string::npos ? line.size() : en) - st;
    if (len) fields.push_back(parse_field(line.data() + st, len));
    if (en == std::string::npos) break;
    st = en + 1;
  }
}

inline ParsedShard parse_lines(const std::vector<std::string>& lines, char sep = ',',
                               int threads = 16) {
  ParsedShard s;
  s.n = (int64_t)lines.size();
  if (s.n == 0) return s;
  std::vector<double> first;
  parse_one_line(lines[0], sep, first);
  if (first.empty()) throw std::invalid_argument("empty sample line");
  s.d = (int64_t)first.size();  // k features + label  ->  bias + k features
  s.X.resize((size_t)s.n * s.d);
  s.y.resize(s.n);
  if (threads < 1) threads = 1;
  if ((int64_t)threads > s.n) threads = (int)s.n;
  std::vector<std::string> errors(threads);
  auto work = [&](int t) {
    std::vector<double> fields;
    const int64_t lo = s.n * t / threads, hi = s.n * (t + 1) / threads;
    try {
      for (int64_t i = lo; i < hi; ++i) {
        parse_one_line(lines[i], sep, fields);
        if ((int64_t)fields.size() != s.d)
          throw std::invalid_argument("ragged sample line " + std::to_string(i));
        double* row = s.X.data() + i * s.d;
        row[0] = 1.;
        for (int64_t j = 0; j + 1 < s.d; ++j) row[j + 1] = fields[j];
        s.y[i] = fields.back();
      }
    } catch (const std::exception& e) {
      errors[t] = e.what();
    }
  };
  std::vector<std::thread> th;
  for (int t = 1; t < threads; ++t) th.emplace_back(work, t);
  work(0);
  for (auto& x : th) x.join();
  for (const std::string& e : errors)
    if (!e.empty()) throw std::invalid_argument(e);
  return s;
}

struct ShardCacheHeader {
  char magic[8];        // "PLRSHARD"
  uint32_t version;     // 1
  uint32_t reserved;
  int64_t n, d;
  int64_t src_size;     // bytes of the text file the shard was parsed from
  int64_t src_mtime_ns;
};

inline std::string cache_path(const std::string& input, int rank, int np) {
  return input + ".plrshard." + std::to_string(rank) + "of" + std::to_string(np);
}

// The cache covers inputs that are one regular file; directories and globs
// are parsed every time (their member list can change under the same name).
inline bool source_stamp(const std::string& input, int64_t& size, int64_t& mtime_ns) {
  struct stat st;
  if (stat(input.c_str(), &st) != 0 || !S_ISREG(st.st_mode)) return false;
  size = (int64_t)st.st_size;
  mtime_ns = (int64_t)st.st_mtim.tv_sec * 1000000000LL + st.st_mtim.tv_nsec;
  return true;
}

inline bool write_cache(const std::string& input, int rank, int np, const ParsedShard& s) {
  ShardCacheHeader h;
  memset(&h, 0, sizeof h);
  memcpy(h.magic, "PLRSHARD", 8);
  h.version = 1;
  h.n = s.n;
  h.d = s.d;
  if (!source_stamp(input, h.src_size, h.src_mtime_ns)) return false;
  const std::string path = cache_path(input, rank, np), tmp = path + ".tmp";
  FILE* f = fopen(tmp.c_str(), "wb");
  if (!f) return false;  // read-only input directory: run without a cache
  bool ok = fwrite(&h, sizeof h, 1, f) == 1;
  ok = ok && (s.X.empty() || fwrite(s.X.data(), sizeof(double), s.X.size(), f) == s.X.size());
  ok = ok && (s.y.empty() || fwrite(s.y.data(), sizeof(double), s.y.size(), f) == s.y.size());
  ok = (fclose(f) == 0) && ok;
  if (ok) ok = rename(tmp.c_str(), path.c_str()) == 0;
  if (!ok) remove(tmp.c_str());
  return ok;
}

// Reads the header only and validates it against the source file.
inline bool open_cache(const std::string& input, int rank, int np, ShardCacheHeader& h,
                       FILE*& f) {
  f = fopen(cache_path(input, rank, np).c_str(), "rb");
  if (!f) return false;
  int64_t size = 0, mtime = 0;
  const bool ok = fread(&h, sizeof h, 1, f) == 1 && memcmp(h.magic, "PLRSHARD", 8) == 0 &&
                  h.version == 1 && h.n >= 0 && h.d >= 1 && source_stamp(input, size, mtime) &&
                  size == h.src_size && mtime == h.src_mtime_ns;
  if (!ok) {
    fclose(f);
    f = nullptr;
  }
  return ok;
}

// A fresh cache mapped read-only: the rows go to the device straight from the
// page cache, without a copy of the shard in the process.
struct MappedShard {
  void* base = nullptr;
  size_t bytes = 0;
  int64_t n = 0, d = 0;
  MappedShard() {}
  MappedShard(const MappedShard&) = delete;
  MappedShard& operator=(const MappedShard&) = delete;
  ~MappedShard() {
    if (base) munmap(base, bytes);
  }
  const double* X() const {
    return reinterpret_cast<const double*>(static_cast<const char*>(base) + sizeof(ShardCacheHeader));
  }
  const double* y() const { return X() + (size_t)n * d; }
};

inline bool map_cache(const std::string& input, int rank, int np, MappedShard& m) {
  ShardCacheHeader h;
  FILE* f = nullptr;
  if (!open_cache(input, rank, np, h, f)) return false;
  struct stat st;
  const size_t want = sizeof h + ((size_t)h.n * h.d + (size_t)h.n) * sizeof(double);
  bool ok = fstat(fileno(f), &st) == 0 && (size_t)st.st_size == want;
  if (ok) {
    void* p = mmap(nullptr, want, PROT_READ, MAP_PRIVATE, fileno(f), 0);
    ok = p != MAP_FAILED;
    if (ok) {
      m.base = p;
      m.bytes = want;
      m.n = h.n;
      m.d = h.d;
    }
  }
  fclose(f);
  return ok;
}

// The cache written slab by slab from rows that live elsewhere (the device):
// rows(r0, m, X, y) fills rows [r0, r0 + m) into X (m x d, dense) and y; false
// aborts.  The shard never exists whole in this process.
template <class Rows>
inline bool write_cache_rows(const std::string& input, int rank, int np, int64_t n, int64_t d,
                             Rows rows, size_t slab_bytes = 64u << 20) {
  ShardCacheHeader h;
  memset(&h, 0, sizeof h);
  memcpy(h.magic, "PLRSHARD", 8);
  h.version = 1;
  h.n = n;
  h.d = d;
  if (!source_stamp(input, h.src_size, h.src_mtime_ns)) return false;
  const std::string path = cache_path(input, rank, np), tmp = path + ".tmp";
  const int fd = open(tmp.c_str(), O_WRONLY | O_CREAT | O_TRUNC, 0644);
  if (fd < 0) return false;  // read-only input directory: run without a cache
  auto put = [fd](const void* p, size_t bytes, size_t at) {
    for (size_t lo = 0; lo < bytes;) {
      const ssize_t w = pwrite(fd, static_cast<const char*>(p) + lo, bytes - lo, (off_t)(at + lo));
      if (w <= 0) return false;
      lo += (size_t)w;
    }
    return true;
  };
  bool ok = put(&h, sizeof h, 0);
  size_t at = sizeof h;
  const int64_t slab = std::max<int64_t>(1, (int64_t)slab_bytes / (d * (int64_t)sizeof(double)));
  // two slab buffers: one is written to the file (a copy into the page cache,
  // ~10 GB/s, more threads do not help) while the next is fetched
  std::vector<double> X[2], y((size_t)n);
  for (auto& x : X) x.resize((size_t)std::min(slab, std::max<int64_t>(n, 1)) * d);
  std::thread writer;
  std::atomic<bool> wrote(true);
  int k = 0;
  for (int64_t r0 = 0; r0 < n && ok; r0 += slab, k ^= 1) {
    const int64_t m = std::min(slab, n - r0);
    const size_t bytes = (size_t)m * d * sizeof(double);
    try {
      ok = rows(r0, m, X[k].data(), y.data() + r0);
    } catch (...) {  // the writer still holds the other buffer and the file
      if (writer.joinable()) writer.join();
      close(fd);
      remove(tmp.c_str());
      throw;
    }
    if (writer.joinable()) writer.join();  // the other buffer is free again
    ok = ok && wrote.load();
    if (ok) {
      const double* src = X[k].data();
      writer = std::thread([&put, &wrote, src, bytes, at]() {
        if (!put(src, bytes, at)) wrote = false;
      });
    }
    at += bytes;
  }
  if (writer.joinable()) writer.join();
  ok = ok && wrote.load() && put(y.data(), (size_t)n * sizeof(double), at);
  ok = (close(fd) == 0) && ok;
  if (ok) ok = rename(tmp.c_str(), path.c_str()) == 0;
  if (!ok) remove(tmp.c_str());
  return ok;
}

inline bool read_cache(const std::string& input, int rank, int np, ParsedShard& s) {
  ShardCacheHeader h;
  FILE* f = nullptr;
  if (!open_cache(input, rank, np, h, f)) return false;
  s.n = h.n;
  s.d = h.d;
  s.X.resize((size_t)h.n * h.d);
  s.y.resize(h.n);
  bool ok = s.X.empty() || fread(s.X.data(), sizeof(double), s.X.size(), f) == s.X.size();
  ok = ok && (s.y.empty() || fread(s.y.data(), sizeof(double), s.y.size(), f) == s.y.size());
  fclose(f);
  return ok;
}

}  // namespace plr_ps
