// The slice of Paracel's worker API (class paralg, reference include/ps.hpp)
// that the logistic-regression worker uses, with the same method names,
// argument meaning and error behaviour, on top of a client that speaks the
// reference's ZeroMQ/msgpack protocol (include/client.hpp).  One worker
// process, one thread; REQ sockets are created lazily per op family and
// strictly alternate send/recv like kvclt's (client.hpp:541-561).
//
// Worker-to-worker collectives are MPI in the reference (paracel_sync =
// MPI_Barrier, ps.hpp:890-892; Comm::allreduce = MPI_Allreduce(SUM),
// utils/comm.hpp:629-636).  Here the workers are plain processes (one shard
// each, sharing the GPU of the box), so the same two collectives run over what
// every worker already has a connection to -- server 0's key-value table, with
// push and pull_multi_check only (two ops whose behaviour on a missing key is
// the same on the reference's server: push creates it, pull_multi_check leaves
// it out of its answer; server.hpp:254-260, kv.hpp:94-103):
//   barrier    worker r pushes the number k of the barrier it has reached
//              under "plr_sync_<r>" (k = 1, 2, ...: all workers call their
//              barriers in the same order, as MPI requires too) and waits
//              until every worker's key reads k or more.  The counters only
//              grow, so nothing has to be removed and the table holds
//              worker_sz such keys however long the job runs.  The push may
//              go out ahead of time (paracel_sync_arrive).
//   allreduce  worker r pushes its value under "plr_ar_<k mod 2>_<r>", barrier,
//              then pulls all worker_sz values (one request) and adds them in rank order --
//              the same bits on every worker.  Two slots suffice: slot k mod 2
//              is written again in call k + 2, behind the barrier of call
//              k + 1, which nobody passes before every worker has read call k.
// A worker that waits longer than sync_timeout_s (PLR_SYNC_TIMEOUT_S in the
// environment, default 1800) for a barrier throws, naming the workers that
// did not arrive: a crashed peer ends the job instead of hanging it.
// A server carries one job at a time (a second job's barriers would find the
// first one's counters).  With one worker both collectives are no-ops.
#pragma once

#include <stdio.h>
#include <stdlib.h>
#include <sys/stat.h>
#include <unistd.h>
#include <zmq.h>

#include <chrono>
#include <fstream>
#include <iostream>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "msgpack_lite.hpp"
#include "shard_io.hpp"

namespace plr_ps {

// kvclt: include/client.hpp.  ports: [0] pull/contains/remove, [1] push,
// [2] update, [3] bupdate/register_bupdate, [4] ssp ints.
class kvclt {
 public:
  kvclt(const std::string& host, const std::vector<std::string>& ports, void* zctx)
      : host_(host), ports_(ports), zctx_(zctx) {
    for (auto& s : socks_) s = nullptr;
  }
  ~kvclt() {
    for (auto s : socks_)
      if (s) zmq_close(s);
  }

  template <class V>
  bool pull(const std::string& key, V& val) {
    return req(0, paste({pack<std::string>("pull"), pack(key)}), val);
  }
  template <class V>
  bool push(const std::string& key, const V& val) {
    if (push_in_flight_ && !push_end()) return false;
    bool stat = false;
    const bool r = req(1, paste({pack<std::string>("push"), pack(key), pack(val)}), stat);
    return r && stat;
  }
  // A push in two halves: the request goes out now, the reply is collected by
  // push_end() (or by the next push) -- the caller does something else while
  // the server stores the value.
  template <class V>
  void push_begin(const std::string& key, const V& val) {
    if (push_in_flight_) (void)push_end();
    send_only(1, paste({pack<std::string>("push"), pack(key), pack(val)}));
    push_in_flight_ = true;
  }
  bool push_end() {
    if (!push_in_flight_) return true;
    push_in_flight_ = false;
    zmq_msg_t m;
    recv_only(1, &m);
    const std::string data((const char*)zmq_msg_data(&m), zmq_msg_size(&m));
    zmq_msg_close(&m);
    return unpack<bool>(data);
  }
  // client.hpp:93-101: the keys of the list that the table holds, with their
  // stored (packed) values -- one round trip for any number of keys
  detail::StrMap pull_multi_check(const std::vector<std::string>& keys) {
    detail::StrMap got;
    req(0, paste({pack<std::string>("pull_multi_check"), pack(keys)}), got);
    return got;
  }
  bool register_bupdate(const std::string& file, const std::string& func) {
    bool stat = false;
    const bool r = req(3, paste({pack<std::string>("register_bupdate"), pack(file), pack(func)}),
                       stat);
    return r && stat;
  }
  template <class V>
  V bupdate(const std::string& key, const V& delta, bool& r) {
    V val;
    r = req(3, paste({pack<std::string>("bupdate"), pack(key), pack(delta)}), val);
    return val;
  }

  // Dense-vector forms of pull and bupdate: the same bytes on the wire, but
  // the vector is encoded straight into the request buffer and decoded
  // straight out of the reply message (no intermediate packed strings), and
  // bupdate's reply -- the new value, which the non-SSP worker unpacks and
  // drops (ps.hpp:753-770) -- is only checked, not decoded.
  bool pull(const std::string& key, std::vector<double>& val) {
    buf_.clear();
    buf_.append(pack<std::string>("pull")).append(kSeparator).append(pack(key));
    zmq_msg_t m;
    roundtrip(0, buf_, &m);
    const char* p = (const char*)zmq_msg_data(&m);
    const size_t n = zmq_msg_size(&m);
    bool ok = !(n == 5 && memcmp(p, "nokey", 5) == 0);
    if (ok) {
      F64ArrayView a;
      if (view_f64_array(p, n, a)) {
        val.resize(a.n);
        if (!detail::dec_f64_run(a.elems, val.data(), a.n))
          val = unpack<std::vector<double> >(std::string(p, n));
      } else {
        val = unpack<std::vector<double> >(std::string(p, n));
      }
    }
    zmq_msg_close(&m);
    return ok;
  }
  bool bupdate_drop(const std::string& key, const std::vector<double>& delta) {
    buf_.clear();
    buf_.append(pack<std::string>("bupdate")).append(kSeparator).append(pack(key));
    buf_.append(kSeparator);
    append_packed(buf_, delta.data(), delta.size());
    zmq_msg_t m;
    roundtrip(3, buf_, &m);
    const bool ok = !(zmq_msg_size(&m) == 5 && memcmp(zmq_msg_data(&m), "nokey", 5) == 0);
    zmq_msg_close(&m);
    return ok;
  }
  bool push_int(const std::string& key, int v) {
    bool stat = true;
    const bool r = req(4, paste({pack<std::string>("push_int"), pack(key), pack(v)}), stat);
    return r && stat;
  }
  // client.hpp:469-480, :495-501
  bool incr_int(const std::string& key, int delta) {
    bool stat = false;
    const bool r = req(4, paste({pack<std::string>("incr_int"), pack(key), pack(delta)}), stat);
    return r && stat;
  }
  bool pull_int(const std::string& key, int& val) {
    return req(4, paste({pack<std::string>("pull_int"), pack(key)}), val);
  }
  bool contains(const std::string& key) {
    bool v = false;
    req(0, paste({pack<std::string>("contains"), pack(key)}), v);
    return v;
  }

 private:
  // one strictly alternating send/recv on the op family's REQ socket; the
  // caller closes *m.  An empty reply is the reference's internal error
  // (client.hpp:551).
  void roundtrip(int port_idx, const std::string& scrip, zmq_msg_t* m) {
    send_only(port_idx, scrip);
    recv_only(port_idx, m);
  }
  void send_only(int port_idx, const std::string& scrip) {
    void*& s = socks_[port_idx];
    if (!s) {
      s = zmq_socket(zctx_, ZMQ_REQ);
      const std::string ep = "tcp://" + host_ + ":" + ports_.at(port_idx);
      if (zmq_connect(s, ep.c_str()) != 0)
        throw std::runtime_error("connect " + ep + ": " + zmq_strerror(zmq_errno()));
    }
    if (zmq_send(s, scrip.data(), scrip.size(), 0) < 0)
      throw std::runtime_error(std::string("zmq_send: ") + zmq_strerror(zmq_errno()));
  }
  void recv_only(int port_idx, zmq_msg_t* m) {
    void* s = socks_[port_idx];
    zmq_msg_init(m);
    if (zmq_msg_recv(m, s, 0) < 0) {
      zmq_msg_close(m);
      throw std::runtime_error(std::string("zmq_recv: ") + zmq_strerror(zmq_errno()));
    }
    if (zmq_msg_size(m) == 0) {
      zmq_msg_close(m);
      throw std::runtime_error("paracel internal error!");
    }
  }
  template <class V>
  bool req(int port_idx, const std::string& scrip, V& val) {
    zmq_msg_t m;
    roundtrip(port_idx, scrip, &m);
    std::string data((const char*)zmq_msg_data(&m), zmq_msg_size(&m));
    zmq_msg_close(&m);
    if (data == "nokey") return false;
    val = unpack<V>(data);
    return true;
  }

  std::string host_;
  std::vector<std::string> ports_;
  void* zctx_;
  void* socks_[5];
  std::string buf_;  // request buffer of the dense forms, reused across rounds
  bool push_in_flight_ = false;
};

class paralg {
 public:
  // hosts_dct_str: "host:p0,p1,p2,p3,p4" per server joined by _PARACEL_
  // (server.hpp:417-435, utils.hpp:80-92).  The LR model lives under one key
  // ("theta"), i.e. on one server (lr.cpp:16-21), so the ring degenerates to
  // server 0 unless more are given; keys are then placed by std::hash modulo.
  paralg(const std::string& hosts_dct_str, const std::string& _output = "", int _rounds = 1,
         int worker_id = 0, int worker_sz = 1)
      : output(_output), rounds(_rounds), rank_(worker_id), nworker_(worker_sz) {
    zctx_ = zmq_ctx_new();
    for (const std::string& one : split_fields(hosts_dct_str)) {
      const size_t c = one.find(':');
      if (c == std::string::npos) throw std::invalid_argument("bad server info: " + one);
      std::vector<std::string> ports;
      size_t st = c + 1;
      for (;;) {
        const size_t en = one.find(',', st);
        ports.push_back(one.substr(st, en == std::string::npos ? en : en - st));
        if (en == std::string::npos) break;
        st = en + 1;
      }
      if (ports.size() != 5) throw std::invalid_argument("server info needs 5 ports: " + one);
      kvm_.emplace_back(new kvclt(one.substr(0, c), ports, zctx_));
    }
    if (kvm_.empty()) throw std::invalid_argument("no server given");
    if (!output.empty()) mkdir(output.c_str(), 0755);
    if (rank_ == 0) kvm_[0]->push_int("worker_sz", nworker_);  // ps.hpp:119-123
    paracel_sync();
  }
  virtual ~paralg() {
    kvm_.clear();
    if (zctx_) zmq_ctx_term(zctx_);
  }

  // ps.hpp:192-197 -> loader::fixload (load/loader.hpp:81-96): this worker's
  // byte range of the file, line-aligned (rule in shard_io.hpp)
  std::vector<std::string> paracel_load(const std::string& fn) {
    std::vector<std::string> lines = load_lines(fn, rank_, nworker_);
    std::cout << "lines got: " << lines.size() << std::endl;  // loader.hpp:93
    return lines;
  }

  // ps.hpp:437-462: blocking pull; a missing key is an error
  template <class V>
  V paracel_read(const std::string& key) {
    V val;
    if (!srv(key).pull(key, val)) {
      std::cerr << "key does not exist" << std::endl;  // ERROR_ABORT only prints
      return V();
    }
    return val;
  }
  // ps.hpp:648-657
  template <class V>
  bool paracel_write(const std::string& key, const V& val) {
    return srv(key).push(key, val);
  }
  // ps.hpp:372-380: every server loads the reducer
  bool paracel_register_bupdate(const std::string& file, const std::string& func) {
    bool r = true;
    for (auto& k : kvm_) r = r && k->register_bupdate(file, func);
    return r;
  }
  // ps.hpp:753-770: blocking; the reply (the new value) is unpacked and dropped
  template <class V>
  bool paracel_bupdate(const std::string& key, const V& delta) {
    bool r = false;
    (void)srv(key).bupdate(key, delta, r);
    return r;
  }
  bool paracel_bupdate(const std::string& key, const std::vector<double>& delta) {
    return srv(key).bupdate_drop(key, delta);
  }
  // ps.hpp:890-892 (MPI_Barrier there): returns once every worker has arrived
  void paracel_sync() {
    if (nworker_ <= 1) return;
    const int k = ++sync_count_;
    if (announced_) {
      announced_ = false;
      if (!kvm_[0]->push_end()) throw std::runtime_error("paracel_sync: push failed");
    } else if (!kvm_[0]->push(sync_key(rank_), k)) {
      throw std::runtime_error("paracel_sync: push failed");
    }
    std::vector<std::string> others;
    for (int r = 0; r < nworker_; ++r)
      if (r != rank_) others.push_back(sync_key(r));
    const auto start = std::chrono::steady_clock::now();
    const auto deadline = start + std::chrono::duration<double>(sync_timeout_s_);
    for (;;) {
      // every other worker's counter in one round trip; a key not pushed yet is left out
      const detail::StrMap got = kvm_[0]->pull_multi_check(others);
      size_t arrived = 0;
      for (const auto& kv : got) arrived += unpack<int>(kv.second) >= k ? 1 : 0;
      if (arrived == others.size()) return;
      const auto now = std::chrono::steady_clock::now();
      if (now > deadline) {
        std::string missing;
        for (int r = 0; r < nworker_; ++r) {
          if (r == rank_) continue;
          bool here = false;
          for (const auto& kv : got) here = here || (kv.first == sync_key(r) && unpack<int>(kv.second) >= k);
          if (!here) missing += (missing.empty() ? "" : ", ") + std::to_string(r);
        }
        throw std::runtime_error("paracel_sync: barrier " + std::to_string(k) + ": worker(s) " +
                                 missing + " did not arrive within " +
                                 std::to_string(sync_timeout_s_) + " s");
      }
      // the first 2 ms poll after poll (a round trip is tens of microseconds), then at ease
      if (now - start > std::chrono::milliseconds(2)) usleep(100);
    }
  }
  // The arrival half of the next paracel_sync(), ahead of time (no counterpart
  // in the reference, whose barrier is MPI's): "whatever the next barrier
  // protects, this worker has done it" -- its counter goes to the server now,
  // without waiting for the reply, and the paracel_sync() that follows only
  // waits for the others.  For a barrier whose purpose is met early: the one
  // between a round's pass and its bupdate (lr.cpp:143) is there so that nobody
  // updates theta before everybody has read it, which is true of a worker as
  // soon as its read has returned.  The next collective after this call must
  // be that paracel_sync() (an allreduce in between throws).
  void paracel_sync_arrive() {
    if (nworker_ <= 1 || announced_) return;
    kvm_[0]->push_begin(sync_key(rank_), sync_count_ + 1);
    announced_ = true;
  }
  void set_sync_timeout(double seconds) { sync_timeout_s_ = seconds; }
  size_t get_worker_id() const { return rank_; }
  size_t get_worker_size() const { return nworker_; }
  // comm.hpp:629-636 (MPI_Allreduce, MPI_SUM): v becomes the sum over all workers
  void allreduce(double& v) {
    if (nworker_ <= 1) return;
    if (announced_) throw std::logic_error("allreduce between paracel_sync_arrive and paracel_sync");
    const std::string base = "plr_ar_" + std::to_string(reduce_count_++ & 1) + "_";
    if (!kvm_[0]->push(base + std::to_string(rank_), v))
      throw std::runtime_error("allreduce: push failed");
    paracel_sync();
    // all values in one round trip, added in rank order whatever order they come in
    std::vector<std::string> keys;
    for (int r = 0; r < nworker_; ++r) keys.push_back(base + std::to_string(r));
    const detail::StrMap got = kvm_[0]->pull_multi_check(keys);
    if (got.size() != keys.size()) throw std::runtime_error("allreduce: a worker's value is missing");
    double sum = 0.;
    for (int r = 0; r < nworker_; ++r)
      for (const auto& kv : got)
        if (kv.first == keys[r]) sum += unpack<double>(kv.second);
    v = sum;
  }
  void allreduce(int& v) {
    double d = (double)v;  // exact: counts of rows
    allreduce(d);
    v = (int)d;
  }

  // ps.hpp:983-1017 / :1308: "<output><prefix><rank>" (truncated, not
  // appended, as with the reference's default append_flag), std::to_string
  // (6 decimals) joined by sep
  void paracel_dump_vector(const std::vector<double>& v, const std::string& prefix,
                           const std::string& sep) {
    std::ofstream os(todir(output) + prefix + std::to_string(rank_));
    for (size_t i = 0; i + 1 < v.size(); ++i) os << std::to_string(v[i]) << sep;
    if (!v.empty()) os << std::to_string(v.back()) << '\n';
  }
  // the (sample, value) form of predictions, ps.hpp:1312-1319:
  // "x0,x1,...,xk:value" per entry
  void paracel_dump_vector(const std::vector<std::pair<std::vector<double>, double> >& v,
                           const std::string& prefix, const std::string& sep) {
    std::ofstream os(todir(output) + prefix + std::to_string(rank_));
    for (size_t i = 0; i < v.size(); ++i) {
      const std::vector<double>& x = v[i].first;
      for (size_t j = 0; j + 1 < x.size(); ++j) os << std::to_string(x[j]) << ',';
      if (!x.empty()) os << std::to_string(x.back());
      os << ':' << std::to_string(v[i].second) << (i + 1 < v.size() ? sep : std::string("\n"));
    }
  }

 protected:
  std::string output;
  int rounds;

 private:
  static std::string todir(const std::string& d) {
    return (d.empty() || d.back() == '/') ? d : d + "/";
  }
  kvclt& srv(const std::string& key) {
    return *kvm_[kvm_.size() == 1 ? 0 : std::hash<std::string>()(key) % kvm_.size()];
  }
  static std::string sync_key(int r) { return "plr_sync_" + std::to_string(r); }
  static double default_sync_timeout() {
    const char* e = getenv("PLR_SYNC_TIMEOUT_S");
    const double v = e ? atof(e) : 0.;
    return v > 0. ? v : 1800.;
  }
  int rank_, nworker_;
  int sync_count_ = 0;
  bool announced_ = false;  // paracel_sync_arrive() has sent the next barrier's counter
  long reduce_count_ = 0;
  double sync_timeout_s_ = default_sync_timeout();
  void* zctx_ = nullptr;
  std::vector<std::unique_ptr<kvclt> > kvm_;
};

}  // namespace plr_ps
