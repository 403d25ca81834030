// Host-side helpers shared by the translation units of libpskv.so.
#ifndef PSKV_HOST_COMMON_H_
#define PSKV_HOST_COMMON_H_
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "pskv/capi.h"

namespace pskv {

// Records the message for pskv_last_error() on this thread and returns `code`.
int set_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

// Whether [ptr, ptr + bytes) lies inside one buffer handed out by pskv_host_alloc (pinned memory).
bool host_pool_owns(const void* ptr, size_t bytes);

// Frees the workspaces of the device's ordered-match context (match.hip); part of pskv_device_trim.
int match_trim(int device);

#define PSKV_HIP(call)                                                                     \
  do {                                                                                     \
    hipError_t e_ = (call);                                                                \
    if (e_ != hipSuccess) {                                                                \
      const int c_ = (e_ == hipErrorOutOfMemory) ? PSKV_ENOMEM : PSKV_EHIP;                \
      return ::pskv::set_error(c_, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), \
                               __FILE__, __LINE__);                                        \
    }                                                                                      \
  } while (0)

// Makes `device` current for the calling thread for the lifetime of the object.
class DeviceGuard {
 public:
  explicit DeviceGuard(int device) : ok_(true), prev_(-1) {
    if (hipGetDevice(&prev_) != hipSuccess) prev_ = -1;
    if (prev_ != device) ok_ = (hipSetDevice(device) == hipSuccess);
  }
  ~DeviceGuard() {
    int cur = -1;
    if (prev_ >= 0 && hipGetDevice(&cur) == hipSuccess && cur != prev_) (void)hipSetDevice(prev_);
  }
  bool ok() const { return ok_; }

 private:
  bool ok_;
  int prev_;
};

inline uint64_t next_pow2(uint64_t x) {
  uint64_t p = 1;
  while (p < x) p <<= 1;
  return p;
}

inline unsigned grid_for(uint64_t items, unsigned per_block, unsigned max_blocks) {
  uint64_t b = (items + per_block - 1) / per_block;
  if (b < 1) b = 1;
  if (b > max_blocks) b = max_blocks;
  return (unsigned)b;
}

}  // namespace pskv
#endif  // PSKV_HOST_COMMON_H_
