/*
 * Driver that runs the REAL ps::KVWorker<float>::DefaultSlicer of the reference
 * (include/ps/kv_app.h:517-572) on caller-supplied arrays. TEST INFRASTRUCTURE ONLY.
 *
 * It is compiled by oracle/Makefile against the headers and the two source
 * files of the reference where they lie (never copied into this repository):
 *   g++ -fno-access-control -I$(REF)/include ref_slicer.cc $(REF)/src/customer.cc
 *       $(REF)/src/postoffice.cc
 * -fno-access-control is what lets this file name the private member function;
 * -ffunction-sections/--gc-sections drop the parts of Postoffice that would need
 * the transport (src/van.cc), which cannot be built without protobuf and zmq.
 * No reference symbol is replaced or stubbed.
 *
 * Only the slicer is covered: the default request handle ends in
 * KVServer::Response -> Van::Send (kv_app.h:460,514), which lives in van.cc.
 */
#include <cstdint>
#include <cstring>
#include <vector>

#include "ps/ps.h"

#if defined(__GNUC__)
#define PSKV_REF_EXPORT __attribute__((visibility("default")))
#else
#define PSKV_REF_EXPORT
#endif

extern "C" {

/* Status: 0 ok, 1 = a CHECK of the reference fired (dmlc::Error). The text of the
 * failed CHECK is copied to err (at most err_cap-1 chars). Outputs as in
 * pskv_oracle_slice, except that val_pos is reported per slice as [val_lo, val_hi)
 * measured as offsets into the vals array. */
PSKV_REF_EXPORT int pskv_ref_default_slicer(const uint64_t* keys, size_t n, const int32_t* lens,
                                            size_t nlens, size_t nvals,
                                            const uint64_t* range_begin,
                                            const uint64_t* range_end, size_t S, uint64_t* key_lo,
                                            uint64_t* key_hi, uint64_t* val_lo, uint64_t* val_hi,
                                            uint8_t* used, char* err, size_t err_cap) {
  using namespace ps;
  // DefaultSlicer reads no member of its object, and constructing a KVWorker would
  // pull in SimpleApp::Response -> Van::Send. The call therefore goes through
  // zeroed, suitably aligned storage that is never constructed or destroyed.
  alignas(KVWorker<float>) static unsigned char storage[sizeof(KVWorker<float>)];
  KVWorker<float>* worker = reinterpret_cast<KVWorker<float>*>(storage);
  KVPairs<float> send;
  std::vector<float> vals(nvals, 0.0f);
  send.keys = SArray<Key>(const_cast<Key*>(keys), n);
  send.vals = SArray<float>(vals.data(), vals.size());
  if (lens && nlens) send.lens = SArray<int>(const_cast<int*>(lens), nlens);
  std::vector<Range> ranges;
  for (size_t i = 0; i < S; ++i) ranges.push_back(Range(range_begin[i], range_end[i]));
  KVWorker<float>::SlicedKVs sliced;
  try {
    worker->DefaultSlicer(send, ranges, &sliced);
  } catch (const dmlc::Error& e) {
    if (err && err_cap) {
      std::strncpy(err, e.what(), err_cap - 1);
      err[err_cap - 1] = 0;
    }
    return 1;
  }
  for (size_t i = 0; i < S; ++i) {
    used[i] = sliced[i].first ? 1 : 0;
    key_lo[i] = key_hi[i] = val_lo[i] = val_hi[i] = 0;
    if (!sliced[i].first) continue;
    const KVPairs<float>& kv = sliced[i].second;
    key_lo[i] = kv.keys.data() - send.keys.data();
    key_hi[i] = key_lo[i] + kv.keys.size();
    val_lo[i] = kv.vals.data() - send.vals.data();
    val_hi[i] = val_lo[i] + kv.vals.size();
  }
  return 0;
}

/* FindRange of the reference, include/ps/sarray.h:281-287 */
PSKV_REF_EXPORT void pskv_ref_find_range(const uint64_t* arr, size_t n, uint64_t lower,
                                         uint64_t upper, uint64_t* begin, uint64_t* end) {
  ps::SArray<uint64_t> a(const_cast<uint64_t*>(arr), n);
  ps::Range r = ps::FindRange(a, lower, upper);
  *begin = r.begin();
  *end = r.end();
}

}  // extern "C"
