// Minimal msgpack codec for the value types that travel between an LR worker
// and the parameter server, in the framing Paracel's packer uses: an 8-byte
// native size_t length followed by the msgpack bytes
// (reference include/packer.hpp:43-51 pack, :62-75 unpack; msgpack-c itself is
// an external dependency of the reference and is not available here, so the
// published msgpack format is restated: str -> fixstr/str8/str16/str32,
// bool -> c2/c3, int -> smallest of fixint/uint8..64/int8..64,
// double -> cb + 8 bytes big-endian, vector -> fixarray/array16/array32).
#pragma once

#include <stdint.h>
#include <string.h>

#include <stdexcept>
#include <string>
#include <vector>

namespace plr_ps {

namespace detail {

inline void put_be(std::string& o, uint64_t v, int bytes) {
  for (int i = bytes - 1; i >= 0; --i) o.push_back((char)((v >> (8 * i)) & 0xff));
}

inline void enc(std::string& o, const std::string& s) {
  const size_t n = s.size();
  if (n < 32) {
    o.push_back((char)(0xa0 | n));
  } else if (n < 256) {
    o.push_back((char)0xd9);
    put_be(o, n, 1);
  } else if (n < 65536) {
    o.push_back((char)0xda);
    put_be(o, n, 2);
  } else {
    o.push_back((char)0xdb);
    put_be(o, n, 4);
  }
  o.append(s);
}

inline void enc(std::string& o, bool b) { o.push_back((char)(b ? 0xc3 : 0xc2)); }

inline void enc(std::string& o, int64_t v) {
  if (v >= 0) {
    if (v < 128) {
      o.push_back((char)v);
    } else if (v < 256) {
      o.push_back((char)0xcc);
      put_be(o, v, 1);
    } else if (v < 65536) {
      o.push_back((char)0xcd);
      put_be(o, v, 2);
    } else if (v < (int64_t(1) << 32)) {
      o.push_back((char)0xce);
      put_be(o, v, 4);
    } else {
      o.push_back((char)0xcf);
      put_be(o, v, 8);
    }
  } else {
    if (v >= -32) {
      o.push_back((char)(0xe0 | (v + 32)));
    } else if (v >= -128) {
      o.push_back((char)0xd0);
      put_be(o, (uint64_t)v, 1);
    } else if (v >= -32768) {
      o.push_back((char)0xd1);
      put_be(o, (uint64_t)v, 2);
    } else if (v >= -(int64_t(1) << 31)) {
      o.push_back((char)0xd2);
      put_be(o, (uint64_t)v, 4);
    } else {
      o.push_back((char)0xd3);
      put_be(o, (uint64_t)v, 8);
    }
  }
}
inline void enc(std::string& o, int v) { enc(o, (int64_t)v); }

inline void enc(std::string& o, double d) {
  uint64_t u;
  memcpy(&u, &d, 8);
  o.push_back((char)0xcb);
  put_be(o, u, 8);
}

// A run of n float64 elements (cb + 8 bytes big-endian each, 9n bytes) in one
// pass without per-byte appends: model vectors are 10^3..10^5 doubles and
// cross the wire twice per round.
inline void enc_f64_run(char* dst, const double* v, size_t n) {
  for (size_t i = 0; i < n; ++i, dst += 9) {
    uint64_t u;
    memcpy(&u, v + i, 8);
    u = __builtin_bswap64(u);
    dst[0] = (char)0xcb;
    memcpy(dst + 1, &u, 8);
  }
}
// false (v partly written) if an element is not tagged float64
inline bool dec_f64_run(const unsigned char* src, double* v, size_t n) {
  for (size_t i = 0; i < n; ++i, src += 9) {
    if (src[0] != 0xcb) return false;
    uint64_t u;
    memcpy(&u, src + 1, 8);
    u = __builtin_bswap64(u);
    memcpy(v + i, &u, 8);
  }
  return true;
}

inline void enc_array_header(std::string& o, size_t n) {
  if (n < 16) {
    o.push_back((char)(0x90 | n));
  } else if (n < 65536) {
    o.push_back((char)0xdc);
    put_be(o, n, 2);
  } else {
    o.push_back((char)0xdd);
    put_be(o, n, 4);
  }
}

inline void enc(std::string& o, const double* v, size_t n) {
  o.reserve(o.size() + 5 + 9 * n);
  enc_array_header(o, n);
  const size_t at = o.size();
  o.resize(at + 9 * n);
  enc_f64_run(&o[at], v, n);
}
inline void enc(std::string& o, const std::vector<double>& v) { enc(o, v.data(), v.size()); }

struct Reader {
  const unsigned char* p;
  const unsigned char* end;
  uint8_t byte() {
    if (p >= end) throw std::runtime_error("msgpack: truncated");
    return *p++;
  }
  uint64_t be(int bytes) {
    uint64_t v = 0;
    for (int i = 0; i < bytes; ++i) v = (v << 8) | byte();
    return v;
  }
};

inline void dec(Reader& r, std::string& s) {
  const uint8_t t = r.byte();
  size_t n;
  if ((t & 0xe0) == 0xa0) n = t & 0x1f;
  else if (t == 0xd9 || t == 0xc4) n = r.be(1);
  else if (t == 0xda || t == 0xc5) n = r.be(2);
  else if (t == 0xdb || t == 0xc6) n = r.be(4);
  else throw std::runtime_error("msgpack: not a string");
  if ((size_t)(r.end - r.p) < n) throw std::runtime_error("msgpack: truncated string");
  s.assign((const char*)r.p, n);
  r.p += n;
}

inline void dec(Reader& r, bool& b) {
  const uint8_t t = r.byte();
  if (t == 0xc3) b = true;
  else if (t == 0xc2) b = false;
  else throw std::runtime_error("msgpack: not a bool");
}

inline bool dec_int_tagged(Reader& r, uint8_t t, int64_t& v) {
  if (t < 0x80) v = t;
  else if (t >= 0xe0) v = (int8_t)t;
  else if (t == 0xcc) v = (int64_t)r.be(1);
  else if (t == 0xcd) v = (int64_t)r.be(2);
  else if (t == 0xce) v = (int64_t)r.be(4);
  else if (t == 0xcf) v = (int64_t)r.be(8);
  else if (t == 0xd0) v = (int8_t)r.be(1);
  else if (t == 0xd1) v = (int16_t)r.be(2);
  else if (t == 0xd2) v = (int32_t)r.be(4);
  else if (t == 0xd3) v = (int64_t)r.be(8);
  else return false;
  return true;
}

inline void dec(Reader& r, int64_t& v) {
  if (!dec_int_tagged(r, r.byte(), v)) throw std::runtime_error("msgpack: not an integer");
}
inline void dec(Reader& r, int& v) {
  int64_t t;
  dec(r, t);
  v = (int)t;
}

inline void dec(Reader& r, double& d) {
  const uint8_t t = r.byte();
  if (t == 0xcb) {
    const uint64_t u = r.be(8);
    memcpy(&d, &u, 8);
  } else if (t == 0xca) {
    const uint32_t u = (uint32_t)r.be(4);
    float f;
    memcpy(&f, &u, 4);
    d = f;
  } else {
    int64_t v;  // msgpack-c converts integers to double on request
    if (!dec_int_tagged(r, t, v)) throw std::runtime_error("msgpack: not a number");
    d = (double)v;
  }
}

inline void dec(Reader& r, std::vector<double>& v) {
  const uint8_t t = r.byte();
  size_t n;
  if ((t & 0xf0) == 0x90) n = t & 0x0f;
  else if (t == 0xdc) n = r.be(2);
  else if (t == 0xdd) n = r.be(4);
  else throw std::runtime_error("msgpack: not an array");
  // every element takes at least one byte: a length the field cannot hold is
  // refused before anything is allocated for it
  if ((size_t)(r.end - r.p) < n) throw std::runtime_error("msgpack: array longer than its field");
  v.resize(n);
  // all-float64 arrays (what a packed vector<double> always is) in one pass;
  // anything else (integers or float32 among the elements) element by element
  if ((size_t)(r.end - r.p) >= 9 * n && dec_f64_run(r.p, v.data(), n)) {
    r.p += 9 * n;
    return;
  }
  for (size_t i = 0; i < n; ++i) dec(r, v[i]);
}

// a list of strings (packer<list_type<str_type>>: an array of str)
inline void enc(std::string& o, const std::vector<std::string>& v) {
  enc_array_header(o, v.size());
  for (const std::string& s : v) enc(o, s);
}
inline void dec(Reader& r, std::vector<std::string>& v) {
  const uint8_t t = r.byte();
  size_t n;
  if ((t & 0xf0) == 0x90) n = t & 0x0f;
  else if (t == 0xdc) n = r.be(2);
  else if (t == 0xdd) n = r.be(4);
  else throw std::runtime_error("msgpack: not an array");
  if ((size_t)(r.end - r.p) < n) throw std::runtime_error("msgpack: array longer than its field");
  v.resize(n);
  for (size_t i = 0; i < n; ++i) dec(r, v[i]);
}

// a dict of key -> stored bytes (packer<dict_type<str_type, str_type>>: a map
// of str to str), kept in the order it was packed in
using StrMap = std::vector<std::pair<std::string, std::string> >;
inline void enc_map_header(std::string& o, size_t n) {
  if (n < 16) {
    o.push_back((char)(0x80 | n));
  } else if (n < 65536) {
    o.push_back((char)0xde);
    put_be(o, n, 2);
  } else {
    o.push_back((char)0xdf);
    put_be(o, n, 4);
  }
}
inline void dec(Reader& r, StrMap& m) {
  const uint8_t t = r.byte();
  size_t n;
  if ((t & 0xf0) == 0x80) n = t & 0x0f;
  else if (t == 0xde) n = r.be(2);
  else if (t == 0xdf) n = r.be(4);
  else throw std::runtime_error("msgpack: not a map");
  if ((size_t)(r.end - r.p) < 2 * n) throw std::runtime_error("msgpack: map longer than its field");
  m.resize(n);
  for (size_t i = 0; i < n; ++i) {
    dec(r, m[i].first);
    dec(r, m[i].second);
  }
}

}  // namespace detail

// bare msgpack bytes of one value
template <class T>
std::string msgpack_bytes(const T& v) {
  std::string o;
  detail::enc(o, v);
  return o;
}

// Paracel's framed form: size_t length + msgpack bytes (packer.hpp:43-51)
template <class T>
std::string pack(const T& v) {
  const std::string body = msgpack_bytes(v);
  const size_t n = body.size();
  std::string s((const char*)&n, sizeof n);
  s.append(body);
  return s;
}

// packer.hpp:62-75
template <class T>
T unpack(const std::string& s) {
  if (s.size() < sizeof(size_t)) throw std::runtime_error("packer: short field");
  size_t n;
  memcpy(&n, s.data(), sizeof n);
  if (s.size() - sizeof n < n) throw std::runtime_error("packer: truncated field");
  detail::Reader r{(const unsigned char*)s.data() + sizeof n,
                   (const unsigned char*)s.data() + sizeof n + n};
  T v;
  detail::dec(r, v);
  return v;
}

// A framed field seen in place as an array of n float64 elements (the packed
// form of vector<double>): elems points at the first cb tag.  False if the
// field is anything else, or shorter than its header claims.  The element
// tags are checked by dec_f64_run when the run is read.
struct F64ArrayView {
  const unsigned char* elems;
  size_t n;
};
inline bool view_f64_array(const char* field, size_t len, F64ArrayView& out) {
  if (len < sizeof(size_t) + 1) return false;
  size_t body;
  memcpy(&body, field, sizeof body);
  if (len - sizeof body < body || body < 1) return false;
  const unsigned char* p = (const unsigned char*)field + sizeof body;
  const unsigned char* end = p + body;
  const uint8_t t = *p++;
  size_t n;
  if ((t & 0xf0) == 0x90) {
    n = t & 0x0f;
  } else if (t == 0xdc) {
    if (end - p < 2) return false;
    n = ((size_t)p[0] << 8) | p[1];
    p += 2;
  } else if (t == 0xdd) {
    if (end - p < 4) return false;
    n = ((size_t)p[0] << 24) | ((size_t)p[1] << 16) | ((size_t)p[2] << 8) | p[3];
    p += 4;
  } else {
    return false;
  }
  if ((size_t)(end - p) != 9 * n) return false;
  out.elems = p;
  out.n = n;
  return true;
}

// Append the framed form of n doubles to a request buffer without an
// intermediate string (same bytes as pack(std::vector<double>)).
inline void append_packed(std::string& o, const double* v, size_t n) {
  const size_t at = o.size();
  o.append(sizeof(size_t), '\0');
  detail::enc(o, v, n);
  const size_t body = o.size() - at - sizeof(size_t);
  memcpy(&o[at], &body, sizeof body);
}

// Request assembly: fields joined by the literal separator
// (include/paracel_types.hpp:49, include/client.hpp:523-539); the server
// splits on it and drops a trailing empty field
// (include/utils/ext_utility.hpp:66-73).
static const char kSeparator[] = "_PARACEL_";

inline std::string paste(const std::vector<std::string>& packed_fields) {
  std::string s;
  for (size_t i = 0; i < packed_fields.size(); ++i) {
    if (i) s.append(kSeparator);
    s.append(packed_fields[i]);
  }
  return s;
}

inline std::vector<std::string> split_fields(const std::string& scrip) {
  std::vector<std::string> out;
  const size_t sl = sizeof(kSeparator) - 1;
  size_t st = 0;
  for (;;) {
    const size_t en = scrip.find(kSeparator, st);
    if (en == std::string::npos) {
      out.push_back(scrip.substr(st));
      break;
    }
    out.push_back(scrip.substr(st, en - st));
    st = en + sl;
  }
  if (!out.empty() && out.back().empty()) out.pop_back();
  return out;
}


// The same split without copying the fields: (pointer, length) pairs into scrip.
struct FieldView {
  const char* p;
  size_t n;
  std::string str() const { return std::string(p, n); }
};
inline void split_field_views(const std::string& scrip, std::vector<FieldView>& out) {
  out.clear();
  const size_t sl = sizeof(kSeparator) - 1;
  size_t st = 0;
  for (;;) {
    const size_t en = scrip.find(kSeparator, st);
    if (en == std::string::npos) {
      out.push_back(FieldView{scrip.data() + st, scrip.size() - st});
      break;
    }
    out.push_back(FieldView{scrip.data() + st, en - st});
    st = en + sl;
  }
  if (!out.empty() && out.back().n == 0) out.pop_back();
}

}  // namespace plr_ps
