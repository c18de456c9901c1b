// A small parameter-server process that speaks Paracel's wire protocol for
// the operations on the logistic-regression path, so that the worker's
// paracel_read / paracel_write / paracel_register_bupdate / paracel_bupdate
// cross a real ZeroMQ REQ/REP boundary with a dlopen'ed reducer.
//
// What it mirrors (reference include/server.hpp): five REP sockets, one
// thread each (:405-459); four run the op dispatcher thrd_exec (:170-402),
// the fifth the integer table thrd_exec_ssp (:114-167); values are stored as
// the packed bytes the client sent (:312-317); bupdate = get -> reducer ->
// set under one global mutex and replies with the new value (:88-100,
// :331-349); a missing key is answered with the raw bytes "nokey" (:237-247);
// the reducer registered on a socket is that socket's thread's state (:173).
// The reference's servers report their ports to a collector process; this one
// prints "host:p0,p1,p2,p3,p4" (the format of utils.hpp:80-92) on stdout.
//
// Dense-vector fast path (not in the reference; same bytes on the wire and in
// the store): requests are split into views instead of copied fields, and a
// bupdate whose stored value and delta are both packed vector<double> of one
// length, under a reducer that exports a "<func>_dense" twin, is folded on
// unpacked doubles and re-encoded into the stored bytes in place -- one
// decode of each operand and one encode instead of the two by-value string
// copies, two unpacks, one pack and two more copies of the packed path.
// --no-dense switches it off (for A/B timing and tests).
//
// Usage: plr_ps_server [--host 127.0.0.1] [--no-dense]   (runs until killed,
// like the reference's start_server, which prun.py ends with killpg)
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <zmq.h>

#include <mutex>
#include <string>
#include <thread>
#include <unordered_map>
#include <vector>

#include "ps_plugin.hpp"

using namespace plr_ps;

static std::unordered_map<std::string, std::string> tbl_store;  // kv_def.hpp:23
static std::unordered_map<std::string, int> ssp_tbl;            // kv_def.hpp:24
static std::mutex store_mutex;                                   // server.hpp:36
static bool dense_enabled = true;

static bool recv_all(void* sock, std::string& out) {
  zmq_msg_t m;
  zmq_msg_init(&m);
  const int rc = zmq_msg_recv(&m, sock, 0);
  if (rc < 0) {
    zmq_msg_close(&m);
    return false;
  }
  out.assign((const char*)zmq_msg_data(&m), zmq_msg_size(&m));
  zmq_msg_close(&m);
  return true;
}

static void reply(void* sock, const std::string& s) { zmq_send(sock, s.data(), s.size(), 0); }

// Fold a packed delta into a packed stored value through the reducer's dense
// twin.  True if done (stored holds the new value, same length as before);
// false if either side is not an all-float64 array or the lengths differ --
// the caller then takes the packed path.  acc/dl are the thread's scratch.
static bool dense_fold(std::string& stored, const FieldView& delta, dense_update_fn f,
                       std::vector<double>& acc, std::vector<double>& dl) {
  F64ArrayView a, b;
  if (!view_f64_array(stored.data(), stored.size(), a) ||
      !view_f64_array(delta.p, delta.n, b) || a.n != b.n)
    return false;
  acc.resize(a.n);
  dl.resize(b.n);
  if (!detail::dec_f64_run(a.elems, acc.data(), a.n) ||
      !detail::dec_f64_run(b.elems, dl.data(), b.n))
    return false;
  f(acc.data(), dl.data(), a.n);
  detail::enc_f64_run(&stored[(const char*)a.elems - stored.data()], acc.data(), a.n);
  return true;
}

static void op_thread(void* sock) {
  update_result update_f;
  dense_update_fn dense_f = nullptr;
  std::vector<double> acc, dl;
  std::string scrip;
  std::vector<FieldView> msg;
  while (recv_all(sock, scrip)) {
    split_field_views(scrip, msg);
    std::string op;
    try {
      op = unpack<std::string>(msg.at(0).str());
      if (op == "contains") {
        std::lock_guard<std::mutex> g(store_mutex);
        reply(sock, pack<bool>(tbl_store.count(unpack<std::string>(msg.at(1).str())) != 0));
      } else if (op == "pull") {
        // the stored bytes go out verbatim; zmq_send copies them, so sending
        // under the lock saves a copy of the value
        std::lock_guard<std::mutex> g(store_mutex);
        auto it = tbl_store.find(unpack<std::string>(msg.at(1).str()));
        if (it != tbl_store.end()) reply(sock, it->second);
        else reply(sock, std::string("nokey"));
      } else if (op == "register_bupdate" || op == "register_update") {
        std::string err;
        if (!load_update_plugin(unpack<std::string>(msg.at(1).str()),
                                unpack<std::string>(msg.at(2).str()), update_f, err, &dense_f)) {
          fprintf(stderr, "%s\n", err.c_str());  // the reference aborts here
          abort();
        }
        reply(sock, pack<bool>(true));
      } else if (op == "push") {
        std::lock_guard<std::mutex> g(store_mutex);
        tbl_store[unpack<std::string>(msg.at(1).str())] = msg.at(2).str();  // stored verbatim
        reply(sock, pack<bool>(true));
      } else if (op == "update" || op == "bupdate") {
        if (msg.size() == 5) {
          std::string err;
          if (!load_update_plugin(unpack<std::string>(msg[3].str()),
                                  unpack<std::string>(msg[4].str()), update_f, err, &dense_f)) {
            fprintf(stderr, "%s\n", err.c_str());
            abort();
          }
        }
        if (!update_f) {
          fprintf(stderr, "bupdate before register_bupdate on this port\n");
          abort();
        }
        {
          std::lock_guard<std::mutex> g(store_mutex);
          const std::string key = unpack<std::string>(msg.at(1).str());
          auto it = tbl_store.find(key);
          if (it == tbl_store.end()) {
            // first update of a missing key = set
            it = tbl_store.emplace(key, msg.at(2).str()).first;
          } else if (!(dense_enabled && dense_f &&
                       dense_fold(it->second, msg.at(2), dense_f, acc, dl))) {
            it->second = update_f(it->second, msg.at(2).str());
          }
          reply(sock, it->second);  // the new value
        }
      } else if (op == "pullall" || op == "pull_multi_check") {
        // server.hpp:261-264: the whole table as one packed map of key -> stored bytes;
        // server.hpp:254-260 with kv.hpp:94-103: the same for the keys of a list that
        // are in the table (a missing key is left out, not an error)
        std::lock_guard<std::mutex> g(store_mutex);
        std::string body;
        if (op == "pullall") {
          detail::enc_map_header(body, tbl_store.size());
          for (const auto& kv : tbl_store) {
            detail::enc(body, kv.first);
            detail::enc(body, kv.second);
          }
        } else {
          const auto keys = unpack<std::vector<std::string> >(msg.at(1).str());
          std::string entries;
          size_t found = 0;
          for (const std::string& k : keys) {
            const auto it = tbl_store.find(k);
            if (it == tbl_store.end()) continue;
            detail::enc(entries, it->first);
            detail::enc(entries, it->second);
            ++found;
          }
          detail::enc_map_header(body, found);
          body.append(entries);
        }
        const size_t len = body.size();
        std::string out((const char*)&len, sizeof len);
        out.append(body);
        reply(sock, out);
      } else if (op == "remove") {
        std::lock_guard<std::mutex> g(store_mutex);
        reply(sock, pack<bool>(tbl_store.erase(unpack<std::string>(msg.at(1).str())) != 0));
      } else if (op == "clear") {
        std::lock_guard<std::mutex> g(store_mutex);
        tbl_store.clear();
        reply(sock, pack<bool>(true));
      } else {
        fprintf(stderr, "plr_ps_server: unsupported op '%s'\n", op.c_str());
        reply(sock, pack<bool>(false));
      }
    } catch (const std::exception& e) {
      fprintf(stderr, "plr_ps_server: bad request (%s)\n", e.what());
      reply(sock, pack<bool>(false));
    }
  }
}

static void ssp_thread(void* sock) {
  std::string scrip;
  while (recv_all(sock, scrip)) {
    std::vector<std::string> msg = split_fields(scrip);
    try {
      const std::string op = unpack<std::string>(msg.at(0));
      if (op == "push_int") {
        std::lock_guard<std::mutex> g(store_mutex);
        ssp_tbl[unpack<std::string>(msg.at(1))] = unpack<int>(msg.at(2));
        reply(sock, pack<bool>(true));
      } else if (op == "pull_int") {
        std::lock_guard<std::mutex> g(store_mutex);
        auto it = ssp_tbl.find(unpack<std::string>(msg.at(1)));
        if (it == ssp_tbl.end()) reply(sock, "nokey");
        else reply(sock, pack<int>(it->second));
      } else if (op == "incr_int") {
        // kv.hpp:108-112: a missing key is not created; server.hpp:136-153
        // answers true either way
        std::lock_guard<std::mutex> g(store_mutex);
        auto it = ssp_tbl.find(unpack<std::string>(msg.at(1)));
        if (it != ssp_tbl.end()) it->second += unpack<int>(msg.at(2));
        reply(sock, pack<bool>(true));
      } else {
        reply(sock, pack<bool>(false));
      }
    } catch (const std::exception& e) {
      reply(sock, pack<bool>(false));
    }
  }
}

int main(int argc, char** argv) {
  std::string host = "127.0.0.1";
  for (int i = 1; i < argc; ++i) {
    if (!strcmp(argv[i], "--host") && i + 1 < argc) host = argv[++i];
    else if (!strcmp(argv[i], "--no-dense")) dense_enabled = false;
  }
  void* ctx = zmq_ctx_new();
  const int kThreads = 5;  // paracel_types.hpp:45 threads_num
  void* socks[kThreads];
  std::string info = host + ":";
  for (int i = 0; i < kThreads; ++i) {
    socks[i] = zmq_socket(ctx, ZMQ_REP);
    const std::string ep = "tcp://" + host + ":*";
    if (zmq_bind(socks[i], ep.c_str()) != 0) {
      fprintf(stderr, "plr_ps_server: bind %s failed: %s\n", ep.c_str(), zmq_strerror(zmq_errno()));
      return 1;
    }
    char bound[256];
    size_t len = sizeof bound;
    zmq_getsockopt(socks[i], ZMQ_LAST_ENDPOINT, bound, &len);
    const char* colon = strrchr(bound, ':');
    info += (i ? "," : "");
    info += (colon ? colon + 1 : "0");
  }
  printf("%s\n", info.c_str());
  fflush(stdout);
  std::vector<std::thread> th;
  for (int i = 0; i < 4; ++i) th.emplace_back(op_thread, socks[i]);
  th.emplace_back(ssp_thread, socks[4]);
  for (auto& t : th) t.join();
  return 0;
}
