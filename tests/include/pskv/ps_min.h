/*
 * A small in-process stand-in for the part of the ps-lite API that surrounds the
 * key-value data path, so that the GPU slicer and the GPU request handle can be
 * driven exactly the way a ps-lite program drives them, without a scheduler or
 * sockets.
 *
 * It keeps the names, argument meaning and failure behaviour of the interface in
 * dmlc/ps-lite (include/ps/kv_app.h, sarray.h, range.h, base.h): a program written
 * against those headers for the push/pull path compiles against this one. What is
 * different is the inside: every worker request is sliced, handed straight to the
 * servers' request handles on the calling thread and answered before Push/Pull
 * returns, so requests are applied in program order (the reference's receive queue
 * does not promise that for equal priorities, threadsafe_pqueue.h:46-53). Workers
 * may run on threads of their own (tests/test_kv_app_multi_workers.cc:64-69 runs two
 * in one process): a server then handles one request at a time, as its receive
 * thread does (customer.cc:54-66), and a worker's requests stay in its program order.
 *
 * There is deliberately no default slicer and no default request handle here:
 * both must be installed (pskv::GpuSlicer / pskv::GpuKVHandle), so nothing in this
 * header computes a slice or a sum on the CPU.
 *
 * Define PSKV_WITH_REAL_PSLITE and include "ps/ps.h" first to use the adapters with
 * the real library instead; then this header must not be included.
 */
#ifndef PSKV_PS_MIN_H_
#define PSKV_PS_MIN_H_
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <functional>
#include <limits>
#include <memory>
#include <mutex>
#include <sstream>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

namespace dmlc {
/* What a failed CHECK throws in ps-lite (include/dmlc/base.h:20-22, logging.h:263-279). */
struct Error : public std::runtime_error {
  explicit Error(const std::string& s) : std::runtime_error(s) {}
};
}  // namespace dmlc

namespace ps {

/* include/ps/base.h:15-18 */
#if USE_KEY32  // (include/ps/base.h:10-16)
using Key = uint32_t;
#else
using Key = uint64_t;
#endif
static const Key kMaxKey = std::numeric_limits<Key>::max();

namespace detail {
inline void Fail(const char* file, int line, const std::string& what) {
  std::ostringstream os;
  os << file << ":" << line << ": Check failed: " << what;
  throw dmlc::Error(os.str());
}
}  // namespace detail
#define PSKV_MIN_CHECK(cond, what)                                    \
  do {                                                                \
    if (!(cond)) ::ps::detail::Fail(__FILE__, __LINE__, (what));      \
  } while (0)

/* include/ps/range.h:12-23 */
class Range {
 public:
  Range() : lo_(0), hi_(0) {}
  Range(uint64_t begin, uint64_t end) : lo_(begin), hi_(end) {}
  uint64_t begin() const { return lo_; }
  uint64_t end() const { return hi_; }
  uint64_t size() const { return hi_ - lo_; }

 private:
  uint64_t lo_, hi_;
};

/* The subset of ps::SArray (include/ps/sarray.h:40-261) the data path touches:
 * shared ownership, zero-copy views, adoption of foreign memory with a deleter. */
template <typename V>
class SArray {
 public:
  SArray() {}
  explicit SArray(size_t n, V fill = 0) { resize(n, fill); }
  explicit SArray(const std::vector<V>& v) { CopyFrom(v.data(), v.size()); }
  /* view over memory the caller keeps alive (sarray.h:94-100 with deletable = false) */
  SArray(V* data, size_t n, bool deletable = false) {
    if (deletable) {
      reset(data, n, [](V* p) { delete[] p; });
    } else {
      reset(data, n, [](V*) {});
    }
  }
  /* reinterpreting, zero-copy conversion (sarray.h:65-81) */
  template <typename W>
  explicit SArray(const SArray<W>& other) { *this = other; }
  template <typename W>
  void operator=(const SArray<W>& other) {
    const size_t bytes = other.size() * sizeof(W);
    PSKV_MIN_CHECK(bytes % sizeof(V) == 0, "cannot be divided");
    n_ = bytes / sizeof(V);
    cap_ = other.capacity() * sizeof(W) / sizeof(V);
    own_ = std::shared_ptr<V>(other.ptr(), reinterpret_cast<V*>(other.data()));
  }

  template <typename Deleter>
  void reset(V* data, size_t n, Deleter del) {  /* sarray.h:162-165 */
    n_ = n;
    cap_ = n;
    own_.reset(data, del);
  }
  void CopyFrom(const V* src, size_t n) {
    resize(n);
    if (n) std::memcpy(data(), src, n * sizeof(V));
  }
  /* growth keeps the old prefix and fills the rest (zero by default, sarray.h:173-189) */
  void resize(size_t n, V fill = 0) {
    const size_t old = n_;
    if (n > cap_) {
      V* fresh = new V[n];
      if (old) std::memcpy(fresh, data(), old * sizeof(V));
      reset(fresh, n, [](V* p) { delete[] p; });
    } else {
      n_ = n;
    }
    for (size_t i = old; i < n; ++i) data()[i] = fill;
  }
  void clear() { reset(static_cast<V*>(nullptr), 0, [](V*) {}); }

  /* zero-copy [begin, end) (sarray.h:248-255) */
  SArray<V> segment(size_t begin, size_t end) const {
    PSKV_MIN_CHECK(end >= begin, "segment: end < begin");
    PSKV_MIN_CHECK(end <= n_, "segment: end > size");
    SArray<V> s;
    s.own_ = std::shared_ptr<V>(own_, data() + begin);
    s.n_ = s.cap_ = end - begin;
    return s;
  }

  bool empty() const { return n_ == 0; }
  size_t size() const { return n_; }
  size_t capacity() const { return cap_; }
  V* data() const { return own_.get(); }
  V* begin() const { return data(); }
  V* end() const { return data() + n_; }
  V front() const { PSKV_MIN_CHECK(n_ > 0, "front() of an empty array"); return data()[0]; }
  V back() const { PSKV_MIN_CHECK(n_ > 0, "back() of an empty array"); return data()[n_ - 1]; }
  V& operator[](size_t i) { return data()[i]; }
  const V& operator[](size_t i) const { return data()[i]; }
  const std::shared_ptr<V>& ptr() const { return own_; }

 private:
  size_t n_ = 0, cap_ = 0;
  std::shared_ptr<V> own_;
};

/* include/ps/kv_app.h:33-45 */
template <typename Val>
struct KVPairs {
  SArray<Key> keys;
  SArray<Val> vals;
  SArray<int> lens;
  int priority = 0;
};

/* include/ps/kv_app.h:375-388 */
struct KVMeta {
  int cmd;
  bool push;
  bool pull;
  int sender;
  int timestamp;
  int customer_id;
};

template <typename Val> class KVServer;
template <typename Val> class KVWorker;

/* Stands where ps::Postoffice stands for the data path: the number of servers, their key
 * ranges (src/postoffice.cc:169-180) and who is registered. One per process. */
class Postoffice {
 public:
  static Postoffice* Get() {
    static Postoffice po;
    return &po;
  }
  /* what DMLC_NUM_SERVER configures in ps-lite (postoffice.cc:23-24) */
  void set_num_servers(int n) {
    PSKV_MIN_CHECK(n > 0, "num_servers > 0");
    num_servers_ = n;
    ranges_.clear();
    for (int i = 0; i < n; ++i)
      ranges_.push_back(Range(kMaxKey / n * i, kMaxKey / n * (i + 1)));
  }
  int num_servers() const { return num_servers_; }
  const std::vector<Range>& GetServerKeyRanges() {
    if (ranges_.empty()) set_num_servers(num_servers_);
    return ranges_;
  }
  /* servers of one app register in creation order: the i-th created is server rank i */
  int AddServer(int app_id, void* server) {
    std::lock_guard<std::mutex> lk(mu_);
    auto& v = servers_[app_id];
    v.push_back(server);
    return static_cast<int>(v.size()) - 1;
  }
  void RemoveServer(int app_id, void* server) {
    std::lock_guard<std::mutex> lk(mu_);
    auto& v = servers_[app_id];
    v.erase(std::remove(v.begin(), v.end(), server), v.end());
  }
  void* server(int app_id, int rank) {
    std::lock_guard<std::mutex> lk(mu_);
    auto it = servers_.find(app_id);
    if (it == servers_.end() || rank >= static_cast<int>(it->second.size())) return nullptr;
    return it->second[rank];
  }
  void AddWorker(int app_id, int customer_id, void* worker) {
    std::lock_guard<std::mutex> lk(mu_);
    workers_[(static_cast<int64_t>(app_id) << 32) | static_cast<uint32_t>(customer_id)] = worker;
  }
  void RemoveWorker(int app_id, int customer_id) {
    std::lock_guard<std::mutex> lk(mu_);
    workers_.erase((static_cast<int64_t>(app_id) << 32) | static_cast<uint32_t>(customer_id));
  }
  void* worker(int app_id, int customer_id) {
    std::lock_guard<std::mutex> lk(mu_);
    auto it = workers_.find((static_cast<int64_t>(app_id) << 32) | static_cast<uint32_t>(customer_id));
    return it == workers_.end() ? nullptr : it->second;
  }
  /* rank -> node id, as in postoffice.h:100-106 */
  static int ServerRankToID(int rank) { return rank * 2 + 8; }
  static int WorkerRankToID(int rank) { return rank * 2 + 9; }

 private:
  Postoffice() {}
  std::mutex mu_;  /* the two registries; workers may be created on threads of their own */
  int num_servers_ = 1;
  std::vector<Range> ranges_;
  std::unordered_map<int, std::vector<void*>> servers_;
  std::unordered_map<int64_t, void*> workers_;
};

/* include/ps/kv_app.h:393-434 */
template <typename Val>
class KVServer {
 public:
  explicit KVServer(int app_id) : app_id_(app_id) { rank_ = Postoffice::Get()->AddServer(app_id, this); }
  virtual ~KVServer() { Postoffice::Get()->RemoveServer(app_id_, this); }

  using ReqHandle =
      std::function<void(const KVMeta& req_meta, const KVPairs<Val>& req_data, KVServer* server)>;
  void set_request_handle(const ReqHandle& request_handle) {
    PSKV_MIN_CHECK(static_cast<bool>(request_handle), "invalid request handle");
    request_handle_ = request_handle;
  }

  /* Delivers the answer to the worker that sent the request (kv_app.h:496-515). */
  void Response(const KVMeta& req, const KVPairs<Val>& res = KVPairs<Val>());

  /* Entry of one request message: what KVServer::Process does with msg.data (kv_app.h:468-494). */
  void Process(const KVMeta& meta, const KVPairs<Val>& data) {
    if (data.lens.size()) PSKV_MIN_CHECK(data.lens.size() == data.keys.size(), "lens.size() == keys.size()");
    PSKV_MIN_CHECK(static_cast<bool>(request_handle_), "no request handle installed");
    std::lock_guard<std::mutex> one_at_a_time(mu_);
    responses_ = 0;
    request_handle_(meta, data, this);
    /* a handle must answer exactly once, or the worker's Wait would hang (customer.cc:32-37) */
    PSKV_MIN_CHECK(responses_ == 1, "the request handle must call Response exactly once");
  }
  int rank() const { return rank_; }
  int app_id() const { return app_id_; }

 private:
  int app_id_, rank_ = 0, responses_ = 0;
  std::mutex mu_;
  ReqHandle request_handle_;
};

/* include/ps/kv_app.h:54-372 */
template <typename Val>
class KVWorker {
 public:
  using Callback = std::function<void()>;
  using SlicedKVs = std::vector<std::pair<bool, KVPairs<Val>>>;
  using Slicer =
      std::function<void(const KVPairs<Val>& send, const std::vector<Range>& ranges, SlicedKVs* sliced)>;

  explicit KVWorker(int app_id, int customer_id) : app_id_(app_id), customer_id_(customer_id) {
    Postoffice::Get()->AddWorker(app_id, customer_id, this);
  }
  virtual ~KVWorker() { Postoffice::Get()->RemoveWorker(app_id_, customer_id_); }

  void set_slicer(const Slicer& slicer) {
    PSKV_MIN_CHECK(static_cast<bool>(slicer), "slicer");
    slicer_ = slicer;
  }

  int Push(const std::vector<Key>& keys, const std::vector<Val>& vals, const std::vector<int>& lens = {},
           int cmd = 0, const Callback& cb = nullptr, int priority = 0) {
    return ZPush(SArray<Key>(keys), SArray<Val>(vals), SArray<int>(lens), cmd, cb, priority);
  }
  int Pull(const std::vector<Key>& keys, std::vector<Val>* vals, std::vector<int>* lens = nullptr,
           int cmd = 0, const Callback& cb = nullptr, int priority = 0) {
    return PullInto(SArray<Key>(keys), SArray<Val>(), vals, lens, false, cmd, cb, priority);
  }
  int PushPull(const std::vector<Key>& keys, const std::vector<Val>& vals, std::vector<Val>* outs,
               std::vector<int>* lens = nullptr, int cmd = 0, const Callback& cb = nullptr,
               int priority = 0) {
    PSKV_MIN_CHECK(outs != nullptr, "outs");
    if (outs->empty()) {
      outs->resize(vals.size());
    } else {
      PSKV_MIN_CHECK(vals.size() == outs->size(), "vals.size() == outs->size()");
    }
    return PullInto(SArray<Key>(keys), SArray<Val>(vals), outs, lens, true, cmd, cb, priority);
  }
  int ZPush(const SArray<Key>& keys, const SArray<Val>& vals, const SArray<int>& lens = SArray<int>(),
            int cmd = 0, const Callback& cb = nullptr, int priority = 0) {
    const int ts = NewRequest();
    KVPairs<Val> kvs;
    kvs.keys = keys;
    kvs.vals = vals;
    kvs.lens = lens;
    kvs.priority = priority;
    Send(ts, true, false, cmd, kvs);
    if (cb) cb();
    return ts;
  }
  int ZPull(const SArray<Key>& keys, SArray<Val>* vals, SArray<int>* lens = nullptr, int cmd = 0,
            const Callback& cb = nullptr, int priority = 0) {
    return PullInto(keys, SArray<Val>(), vals, lens, false, cmd, cb, priority);
  }
  int ZPushPull(const SArray<Key>& keys, const SArray<Val>& vals, SArray<Val>* outs,
                SArray<int>* lens = nullptr, int cmd = 0, const Callback& cb = nullptr,
                int priority = 0) {
    return PullInto(keys, vals, outs, lens, true, cmd, cb, priority);
  }
  /* Requests complete before they return here; Wait only checks the timestamp. */
  void Wait(int timestamp) { PSKV_MIN_CHECK(timestamp >= 0 && timestamp < next_ts_, "unknown timestamp"); }

  /* called by KVServer::Response */
  void Receive(int timestamp, const KVPairs<Val>& res) {
    if (res.keys.size()) received_[timestamp].push_back(res);
  }
  int customer_id() const { return customer_id_; }

 private:
  int NewRequest() { return next_ts_++; }

  /* kv_app.h:574-613 without the wire: one request per non-empty slice, in server order */
  void Send(int timestamp, bool push, bool pull, int cmd, const KVPairs<Val>& kvs) {
    PSKV_MIN_CHECK(static_cast<bool>(slicer_), "no slicer installed (KVWorker::set_slicer)");
    SlicedKVs sliced;
    slicer_(kvs, Postoffice::Get()->GetServerKeyRanges(), &sliced);
    for (size_t i = 0; i < sliced.size(); ++i) {
      if (!sliced[i].first) continue;
      auto* server = static_cast<KVServer<Val>*>(Postoffice::Get()->server(app_id_, static_cast<int>(i)));
      PSKV_MIN_CHECK(server != nullptr, "no server for a non-empty slice");
      KVMeta meta;
      meta.cmd = cmd;
      meta.push = push;
      meta.pull = pull;
      meta.sender = Postoffice::WorkerRankToID(0);
      meta.timestamp = timestamp;
      meta.customer_id = customer_id_;
      server->Process(meta, sliced[i].second);
    }
  }

  /* The pull callback of kv_app.h:663-714: per-server answers are matched against the request
   * keys, ordered by first key and copied into the caller's buffers. */
  template <typename C, typename D>
  int PullInto(const SArray<Key>& keys, const SArray<Val>& push_vals, C* vals, D* lens, bool push,
               int cmd, const Callback& cb, int priority) {
    const int ts = NewRequest();
    KVPairs<Val> kvs;
    kvs.keys = keys;
    kvs.priority = priority;
    if (push) {
      kvs.vals = push_vals;
      if (lens) kvs.lens = SArray<int>(lens->data(), lens->size());
    }
    Send(ts, push, true, cmd, kvs);
    std::vector<KVPairs<Val>>& got = received_[ts];
    size_t total_key = 0, total_val = 0;
    for (const auto& s : got) {
      const Key lo = s.keys.front(), hi = s.keys.back() + 1;
      size_t cnt = 0;
      if (hi > lo) {
        cnt = std::lower_bound(keys.begin(), keys.end(), hi) - std::lower_bound(keys.begin(), keys.end(), lo);
      }
      PSKV_MIN_CHECK(cnt == s.keys.size(), "unmatched keys size from one server");
      if (lens) PSKV_MIN_CHECK(s.lens.size() == s.keys.size(), "lens missing in a pull response");
      total_key += s.keys.size();
      total_val += s.vals.size();
    }
    PSKV_MIN_CHECK(total_key == keys.size(), "lost some servers?");
    std::sort(got.begin(), got.end(),
              [](const KVPairs<Val>& a, const KVPairs<Val>& b) { return a.keys.front() < b.keys.front(); });
    PSKV_MIN_CHECK(vals != nullptr, "vals");
    if (vals->empty()) {
      vals->resize(total_val);
    } else {
      PSKV_MIN_CHECK(vals->size() == total_val, "vals->size() == total_val");
    }
    if (lens) {
      if (lens->empty()) {
        lens->resize(keys.size());
      } else {
        PSKV_MIN_CHECK(lens->size() == keys.size(), "lens->size() == keys.size()");
      }
    }
    Val* pv = vals->data();
    int* pl = lens ? lens->data() : nullptr;
    for (const auto& s : got) {
      if (s.vals.size()) std::memcpy(pv, s.vals.data(), s.vals.size() * sizeof(Val));
      pv += s.vals.size();
      if (pl) {
        std::memcpy(pl, s.lens.data(), s.lens.size() * sizeof(int));
        pl += s.lens.size();
      }
    }
    received_.erase(ts);
    if (cb) cb();
    return ts;
  }

  int app_id_, customer_id_;
  int next_ts_ = 0;
  Slicer slicer_;
  std::unordered_map<int, std::vector<KVPairs<Val>>> received_;
};

template <typename Val>
void KVServer<Val>::Response(const KVMeta& req, const KVPairs<Val>& res) {
  ++responses_;
  auto* w = static_cast<KVWorker<Val>*>(Postoffice::Get()->worker(app_id_, req.customer_id));
  PSKV_MIN_CHECK(w != nullptr, "response for an unknown worker");
  w->Receive(req.timestamp, res);
}

}  // namespace ps
#endif  // PSKV_PS_MIN_H_
