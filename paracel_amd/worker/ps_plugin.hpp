// The parameter server's reducer plugin ABI, as the reference defines it: a
// shared object exports, with C linkage, a GLOBAL OBJECT of type
// std::function<std::string(std::string, std::string)> taking the packed old
// value and the packed delta and returning the packed new value
// (reference include/proxy.hpp:28,56-73; alg/.../update.cpp:22-24,34).  The
// server dlopens the file, copies the std::function by value and dlcloses
// (include/server.hpp:177-191).
#pragma once

#include <dlfcn.h>

#include <functional>
#include <string>

#include "msgpack_lite.hpp"

namespace plr_ps {

typedef std::function<std::string(std::string, std::string)> update_result;

// Wrap a typed reducer V f(V, V) into the packed-string form (proxy.hpp:56-73).
template <class V>
update_result update_proxy(V (*func)(V, V)) {
  return [func](std::string s_val, std::string s_delta) {
    return pack<V>(func(unpack<V>(s_val), unpack<V>(s_delta)));
  };
}

// Optional dense twin of a reducer over vector<double>: a plain C function
// named "<symbol>_dense" in the same shared object that folds `delta` into
// `acc` (both n doubles) and must give, element for element, what the packed
// reducer gives.  Not part of the reference's plugin ABI: a plugin without it
// works as before; with it the server skips the string copies and the
// msgpack round trip of the packed form (three encodes/decodes of the whole
// vector per bupdate in the reference, server.hpp:331-349 + proxy.hpp:56-73).
typedef void (*dense_update_fn)(double* acc, const double* delta, size_t n);

// dlopen(RTLD_NOW|RTLD_LOCAL|RTLD_NODELETE) -> dlsym -> copy -> dlclose.
// Returns false (and fills err) if the file or the symbol is missing.
// dense (nullable) receives the twin, or nullptr if the plugin has none; the
// object stays mapped (RTLD_NODELETE), so the pointer outlives the dlclose.
inline bool load_update_plugin(const std::string& file, const std::string& symbol,
                               update_result& out, std::string& err,
                               dense_update_fn* dense = nullptr) {
  void* h = dlopen(file.c_str(), RTLD_NOW | RTLD_LOCAL | RTLD_NODELETE);
  if (!h) {
    err = std::string("Cannot open library: ") + dlerror();
    return false;
  }
  void* sym = dlsym(h, symbol.c_str());
  if (!sym) {
    err = std::string("Cannot load symbol: ") + dlerror();
    dlclose(h);
    return false;
  }
  out = *reinterpret_cast<update_result*>(sym);
  if (dense) *dense = reinterpret_cast<dense_update_fn>(dlsym(h, (symbol + "_dense").c_str()));
  dlclose(h);
  return true;
}

}  // namespace plr_ps
