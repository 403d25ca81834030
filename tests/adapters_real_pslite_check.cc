// Compile-only proof that the adapters fit the REAL ps-lite extension points: built with
// -I<ps-lite>/include by tests/test_boundary.py where the reference tree is present.
#include <functional>
#include <type_traits>

#include "ps/ps.h"
#include "pskv/ps_adapters.h"

static_assert(std::is_constructible<ps::KVWorker<float>::Slicer, pskv::GpuSlicer<float>>::value,
              "GpuSlicer must be installable with KVWorker::set_slicer");
static_assert(std::is_constructible<ps::KVServer<float>::ReqHandle, pskv::GpuKVHandle<float>>::value,
              "GpuKVHandle must be installable with KVServer::set_request_handle");
static_assert(std::is_copy_constructible<pskv::GpuKVHandle<float>>::value,
              "set_request_handle copies the functor");

// instantiate every member against the real SArray / KVPairs / KVServer
template class pskv::GpuSlicer<float>;
template class pskv::GpuKVHandle<float>;

void install(ps::KVWorker<float>* w, ps::KVServer<float>* s) {
  w->set_slicer(pskv::GpuSlicer<float>(0));
  s->set_request_handle(pskv::GpuKVHandle<float>());
}

// the ordered match with the reference's containers on both ends (parallel_kv_match.h:95-100)
size_t merge(const ps::SArray<ps::Key>& src_key, const ps::SArray<float>& src_val,
             const ps::SArray<ps::Key>& dst_key, ps::SArray<float>* into_sarray, std::vector<float>* into_vector) {
  return pskv::GpuOrderedMatch(src_key, src_val, dst_key, into_sarray, 2, PSKV_OP_PLUS) +
         pskv::GpuOrderedMatch(src_key, src_val, dst_key, into_vector);
}
