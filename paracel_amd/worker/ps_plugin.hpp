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

// dlopen(RTLD_NOW|RTLD_LOCAL|RTLD_NODELETE) -> dlsym -> copy -> dlclose.
// Returns false (and fills err) if the file or the symbol is missing.
inline bool load_update_plugin(const std::string& file, const std::string& symbol,
                               update_result& out, std::string& err) {
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
  dlclose(h);
  return true;
}

}  // namespace plr_ps
