/*
 * Drop-in adapters between ps-lite's two extension points on the key-value data
 * path and the pskv C ABI (pskv/capi.h):
 *
 *   pskv::GpuSlicer<Val>    has the signature of ps::KVWorker<Val>::Slicer
 *                           (include/ps/kv_app.h:315-317) and replaces
 *                           KVWorker::DefaultSlicer (kv_app.h:517-572);
 *                           install with KVWorker::set_slicer (kv_app.h:322-324).
 *   pskv::GpuKVHandle<Val>  has the signature of ps::KVServer<Val>::ReqHandle
 *                           (kv_app.h:414-416) and replaces KVServerDefaultHandle
 *                           (kv_app.h:440-463); install with
 *                           KVServer::set_request_handle (kv_app.h:417-420).
 *
 * Include the real library ("ps/ps.h") BEFORE this header (the tests of this repository
 * include their in-process stand-in, tests/include/pskv/ps_min.h, instead);
 * it only uses names both provide (ps::KVPairs, ps::KVMeta, ps::KVServer,
 * ps::KVWorker, ps::Range, ps::SArray, dmlc::Error).
 *
 * Failure convention: where the reference would fail a CHECK and throw
 * dmlc::Error (include/dmlc/logging.h:263-279), the adapters throw dmlc::Error
 * with the text of pskv_last_error(). The C ABI itself never throws.
 */
#ifndef PSKV_PS_ADAPTERS_H_
#define PSKV_PS_ADAPTERS_H_
#include <cstdint>
#include <memory>
#include <string>
#include <type_traits>
#include <vector>

#include "pskv/capi.h"

namespace pskv {

inline void ThrowStatus(int rc, const char* where) {
  throw dmlc::Error(std::string(where) + ": " + pskv_last_error() + " (status " + std::to_string(rc) + ")");
}

namespace detail {
/* The C ABI takes 64-bit keys. A ps-lite built with USE_KEY32 (include/ps/base.h:10-16) has 32-bit
 * keys: the adapters widen them into a buffer of their own for the duration of the call (order,
 * uniqueness and the key ranges of Postoffice::GetServerKeyRanges, which are uint64_t either way,
 * are kept; responses share the request's own key buffer, kv_app.h:449, so nothing is narrowed). */
template <typename K, bool kNative = sizeof(K) == 8>
struct Keys64;
template <typename K>
struct Keys64<K, true> {
  Keys64(const K* p, size_t) : ptr(reinterpret_cast<const uint64_t*>(p)) {}
  const uint64_t* ptr;
};
template <typename K>
struct Keys64<K, false> {
  static_assert(sizeof(K) == 4, "ps::Key is 32 or 64 bits wide");
  Keys64(const K* p, size_t n) : buf(n) {
    for (size_t i = 0; i < n; ++i) buf[i] = static_cast<uint64_t>(p[i]);
    ptr = buf.data();
  }
  std::vector<uint64_t> buf;
  const uint64_t* ptr;
};
}  // namespace detail

/* The KVWorker::Slicer that runs the boundary search and the lens sums on the GPU.
 * Copyable and re-entrant (KVWorker::Push may be called from several threads,
 * kv_app.h:101-104). The slices are zero-copy segments of the request, exactly like
 * the reference's (SArray::segment, sarray.h:248-255). */
template <typename Val>
class GpuSlicer {
 public:
  using SlicedKVs = typename ps::KVWorker<Val>::SlicedKVs;
  explicit GpuSlicer(int device = 0) : device_(device) {}

  void operator()(const ps::KVPairs<Val>& send, const std::vector<ps::Range>& ranges,
                  SlicedKVs* sliced) const {
    const size_t S = ranges.size();
    sliced->resize(S);  // kv_app.h:521
    std::vector<uint64_t> rb(S), re(S), pos(S + 1), val_pos(S + 1);
    std::vector<uint8_t> used(S ? S : 1);
    for (size_t i = 0; i < S; ++i) {
      rb[i] = ranges[i].begin();
      re[i] = ranges[i].end();
    }
    const detail::Keys64<ps::Key> keys(send.keys.data(), send.keys.size());
    const int rc = pskv_slice(device_, keys.ptr, send.keys.size(),
                              reinterpret_cast<const int32_t*>(send.lens.data()), send.lens.size(),
                              send.vals.size(), rb.data(), re.data(), S, pos.data(), val_pos.data(),
                              used.data(), PSKV_MEM_HOST);
    if (rc != PSKV_OK) ThrowStatus(rc, "GpuSlicer");
    for (size_t i = 0; i < S; ++i) {  // kv_app.h:555-571
      sliced->at(i).first = used[i] != 0;
      if (!used[i]) continue;
      ps::KVPairs<Val>& kv = sliced->at(i).second;
      kv.keys = send.keys.segment(pos[i], pos[i + 1]);
      if (send.lens.size()) kv.lens = send.lens.segment(pos[i], pos[i + 1]);
      kv.vals = send.vals.segment(val_pos[i], val_pos[i + 1]);
    }
  }

 private:
  int device_;
};

/* The KVServer::ReqHandle whose store lives in HBM. The functor is copied into a
 * std::function by set_request_handle (the reference passes a temporary that owns the
 * store, tests/test_kv_app.cc:11), so copies share one table.
 *
 * opts.mode selects what a key holds: PSKV_MODE_SCALAR is the drop-in for
 * KVServerDefaultHandle<float>; PSKV_MODE_FIXED / PSKV_MODE_VARLEN store the
 * multi-float layouts of KVPairs (kv_app.h:17-31), which the reference's default
 * handle rejects (kv_app.h:447).
 *
 * Must be called from one thread at a time, which is how KVServer calls it (the
 * Customer receive thread, src/customer.cc:49-63). Calls Response exactly once per
 * request, after the device work of the request is complete. Pull responses are
 * returned in pinned host buffers that go back to a pool when the last SArray copy
 * dies, on whatever thread that happens. */
template <typename Val>
class GpuKVHandle {
  static_assert(std::is_same<Val, float>::value, "the GPU store holds float32 values");

 public:
  explicit GpuKVHandle(const pskv_opts& opts) : table_(Create(opts)), mode_(opts.mode) {}
  GpuKVHandle() : GpuKVHandle(DefaultOpts()) {}

  void operator()(const ps::KVMeta& req_meta, const ps::KVPairs<Val>& req_data, ps::KVServer<Val>* server) {
    const size_t n = req_data.keys.size();
    const detail::Keys64<ps::Key> wide(req_data.keys.data(), n);
    const uint64_t* keys = wide.ptr;
    const float* vals = req_data.vals.data();
    const int32_t* lens = reinterpret_cast<const int32_t*>(req_data.lens.data());
    const size_t nlens = mode_ == PSKV_MODE_VARLEN ? req_data.lens.size() : 0;
    ps::KVPairs<Val> res;
    if (!req_meta.pull) {
      if (req_meta.push) {
        const int rc = pskv_push(table_.get(), keys, n, vals, req_data.vals.size(), lens, nlens, PSKV_MEM_HOST);
        if (rc != PSKV_OK) ThrowStatus(rc, "GpuKVHandle push");
      } else if (n != req_data.vals.size()) {
        // neither push nor pull: the reference still checks the sizes (kv_app.h:446-447)
        throw dmlc::Error("GpuKVHandle: Check failed: n == req_data.vals.size()");
      }
      server->Response(req_meta, res);  // kv_app.h:460 with an empty res
      return;
    }
    // pull, or push+pull: size the response, run, hand the pinned buffers to SArrays
    size_t need = 0;
    float* out = nullptr;
    int32_t* out_lens = nullptr;
    size_t cap = ResponseGuess(n, req_data);
    for (int attempt = 0; attempt < 2; ++attempt) {
      out = static_cast<float*>(pskv_host_alloc((cap ? cap : 1) * sizeof(float)));
      if (mode_ == PSKV_MODE_VARLEN && !out_lens)
        out_lens = static_cast<int32_t*>(pskv_host_alloc((n ? n : 1) * sizeof(int32_t)));
      if (!out || (mode_ == PSKV_MODE_VARLEN && !out_lens)) ThrowStatus(PSKV_ENOMEM, "GpuKVHandle");
      int rc;
      if (req_meta.push && attempt == 0) {
        rc = pskv_pushpull(table_.get(), keys, n, vals, req_data.vals.size(), lens, nlens, out, cap, out_lens,
                           &need, PSKV_MEM_HOST);
      } else {
        // the push half of a push+pull was applied by the first attempt
        rc = pskv_pull(table_.get(), keys, n, out, cap, out_lens, &need, PSKV_MEM_HOST);
      }
      if (rc == PSKV_OK) break;
      pskv_host_free(out);
      out = nullptr;
      if (rc == PSKV_ESIZE_MISMATCH && need > cap && attempt == 0) {
        cap = need;  // only a var-len response can be larger than the guess
        continue;
      }
      pskv_host_free(out_lens);
      ThrowStatus(rc, "GpuKVHandle pull");
    }
    last_response_ = need;
    res.keys = req_data.keys;  // kv_app.h:449: the response shares the request's key buffer
    res.vals.reset(out, need, [](Val* p) { pskv_host_free(p); });
    if (out_lens) {
      res.lens.reset(reinterpret_cast<int*>(out_lens), n, [](int* p) { pskv_host_free(p); });
    }
    server->Response(req_meta, res);
  }

  pskv_table* table() const { return table_.get(); }

 private:
  static pskv_opts DefaultOpts() {
    pskv_opts o = pskv_opts();
    o.mode = PSKV_MODE_SCALAR;
    return o;
  }
  static std::shared_ptr<pskv_table> Create(const pskv_opts& opts) {
    pskv_table* t = nullptr;
    const int rc = pskv_table_create(&t, &opts);
    if (rc != PSKV_OK) ThrowStatus(rc, "GpuKVHandle");
    return std::shared_ptr<pskv_table>(t, [](pskv_table* p) { pskv_table_destroy(p); });
  }
  size_t ResponseGuess(size_t n, const ps::KVPairs<Val>& req) const {
    if (mode_ == PSKV_MODE_SCALAR) return n;
    if (req.vals.size()) return req.vals.size();  // push+pull answers what was pushed
    return n ? last_response_ : 0;                // var-len / fixed pull: start from the last size
  }

  std::shared_ptr<pskv_table> table_;
  int mode_;
  size_t last_response_ = 0;
};

/* ParallelOrderedMatch (include/ps/internal/parallel_kv_match.h:95-120) on the GPU, with the
 * reference's parameter order: merges src_val into *dst_val where the sorted unique keys are
 * equal, `dst_val[i] op= src_val[j]`, k values per key. *dst_val is resized to
 * dst_key.size() * k first (new entries are zero, :109), as the reference does. `op` is one of
 * PSKV_OP_ASSIGN .. PSKV_OP_DIVIDE, numbered like ps::AssignOp (assign_op.h:12-21); the
 * reference's thread count has no meaning here. Returns the number of matched values. C is
 * ps::SArray<Val> or std::vector<Val>. */
template <typename Val, typename C>
size_t GpuOrderedMatch(const ps::SArray<ps::Key>& src_key, const ps::SArray<Val>& src_val,
                       const ps::SArray<ps::Key>& dst_key, C* dst_val, int k = 1, int op = PSKV_OP_ASSIGN,
                       int device = 0) {
  static_assert(sizeof(Val) == 4, "float values");
  if (k <= 0 || src_key.size() * static_cast<size_t>(k) != src_val.size())  // CHECK_EQ, :107
    throw dmlc::Error("GpuOrderedMatch: Check failed: src_key.size() * k == src_val.size()");
  dst_val->resize(dst_key.size() * static_cast<size_t>(k));  // :109
  if (dst_key.empty()) return 0;
  uint64_t matched = 0;
  const detail::Keys64<ps::Key> src(src_key.data(), src_key.size()), dst(dst_key.data(), dst_key.size());
  const int rc = pskv_match(device, src.ptr, src_key.size(), reinterpret_cast<const float*>(src_val.data()),
                            dst.ptr, dst_key.size(),
                            reinterpret_cast<float*>(dst_val->data()), static_cast<size_t>(k), op, &matched,
                            nullptr, PSKV_MEM_HOST);
  if (rc != PSKV_OK) ThrowStatus(rc, "GpuOrderedMatch");
  return static_cast<size_t>(matched);
}

}  // namespace pskv
#endif  // PSKV_PS_ADAPTERS_H_
