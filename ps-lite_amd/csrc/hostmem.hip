// Pinned host buffers for request and response staging.
//
// A ps-lite response SArray is released on a transport thread once the message
// has been sent (src/zmq_van.h:20-26,159-175), so giving a buffer back must be
// thread-safe and must not block in the HIP runtime: pskv_host_free only pushes
// the buffer onto a free list; pskv_host_trim (any thread, any time) is what
// returns memory to the system.
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "host_common.h"

namespace {

struct Pool {
  std::mutex mu;
  std::map<size_t, std::vector<void*>> free_by_size;  // size class -> buffers
  std::unordered_map<void*, size_t> size_of;          // every live allocation
};

Pool& pool() {
  static Pool* p = new Pool();  // never destroyed: buffers may be freed during process exit
  return *p;
}

size_t size_class(size_t bytes) {
  size_t c = 4096;
  while (c < bytes) c <<= 1;
  return c;
}

}  // namespace

extern "C" {

void* pskv_host_alloc(size_t bytes) {
  const size_t c = size_class(bytes ? bytes : 1);
  Pool& p = pool();
  {
    std::lock_guard<std::mutex> lk(p.mu);
    auto it = p.free_by_size.find(c);
    if (it != p.free_by_size.end() && !it->second.empty()) {
      void* r = it->second.back();
      it->second.pop_back();
      return r;
    }
  }
  void* r = nullptr;
  if (hipHostMalloc(&r, c, hipHostMallocDefault) != hipSuccess) {
    pskv::set_error(PSKV_ENOMEM, "hipHostMalloc of %zu bytes failed", c);
    return nullptr;
  }
  std::lock_guard<std::mutex> lk(p.mu);
  p.size_of[r] = c;
  return r;
}

void pskv_host_free(void* ptr) {
  if (!ptr) return;
  Pool& p = pool();
  std::lock_guard<std::mutex> lk(p.mu);
  auto it = p.size_of.find(ptr);
  if (it == p.size_of.end()) return;  // not ours
  p.free_by_size[it->second].push_back(ptr);
}

}  // extern "C"

namespace pskv {
// Whether [ptr, ptr + bytes) lies inside one buffer of the pinned pool: such memory needs no
// staging, the copy engines reach it directly.
bool host_pool_owns(const void* ptr, size_t bytes) {
  Pool& p = pool();
  const uintptr_t a = reinterpret_cast<uintptr_t>(ptr);
  std::lock_guard<std::mutex> lk(p.mu);
  for (const auto& kv : p.size_of) {  // a handful of live buffers per process
    const uintptr_t base = reinterpret_cast<uintptr_t>(kv.first);
    if (a >= base && a + bytes <= base + kv.second) return true;
  }
  return false;
}
}  // namespace pskv

extern "C" {

int pskv_host_trim(void) {
  Pool& p = pool();
  std::vector<void*> victims;
  {
    std::lock_guard<std::mutex> lk(p.mu);
    for (auto& kv : p.free_by_size) {
      for (void* b : kv.second) {
        victims.push_back(b);
        p.size_of.erase(b);
      }
      kv.second.clear();
    }
  }
  int rc = PSKV_OK;
  for (void* b : victims) {
    if (hipHostFree(b) != hipSuccess) rc = pskv::set_error(PSKV_EHIP, "hipHostFree failed");
  }
  return rc;
}

}  // extern "C"
