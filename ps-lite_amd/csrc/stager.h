// Staging of large host-resident requests and responses.
//
// A ps-lite server receives requests in ordinary host memory (the transport's receive buffers,
// src/zmq_van.h:179-227; KVServer::Process hands them over as they are, include/ps/kv_app.h:468-494)
// and answers into host memory. The copy engines of the GPU only reach pinned memory at full
// speed, so a large transfer goes through a ring of pinned pieces, and the three stages of
// every piece overlap with those of its neighbours:
//   host -> device:  worker threads copy piece c+1 into the ring while piece c is in flight to
//                    the GPU and the kernel that consumes piece c-1 runs;
//   device -> host:  the kernel that produces piece c+1 runs while piece c is in flight to the
//                    ring and worker threads copy piece c-1 to the caller's buffer.
#ifndef PSKV_STAGER_H_
#define PSKV_STAGER_H_
#include <hip/hip_runtime.h>
#include <stddef.h>

#include <functional>

namespace pskv {

class Stager {
 public:
  static constexpr size_t kPiece = 8u << 20;  // bytes per piece of the ring
  static constexpr int kSlots = 16;           // pieces in the ring (128 MiB of pinned memory)
  static constexpr int kSlack = 3;            // slots kept between the piece being sent and the next refill
  static constexpr int kWorkers = 8;          // threads that copy between caller memory and the ring
  static constexpr int kParts = 4;            // a piece is copied in this many parts, by as many workers

  // The stager of `device`, created on first use and kept until the process ends; nullptr when
  // its pinned memory cannot be had (the caller then falls back to plain copy commands).
  static Stager* get(int device);

  // Copies `bytes` from ordinary host memory `src` to device memory `dst`. Piece by piece, in
  // order: once piece c is on its way, `consumer` has been made to wait for it and
  // `after_piece(offset, len)` is called on the calling thread (it may enqueue the work that
  // consumes those bytes on `consumer`; it may be empty). Returns a PSKV_* status.
  int to_device(void* dst, const void* src, size_t bytes, hipStream_t consumer,
                const std::function<int(size_t, size_t)>& after_piece);

  // Copies `bytes` from device memory `src` to ordinary host memory `dst`. Piece by piece, in
  // order: `before_piece(offset, len)` is called on the calling thread (it may enqueue the work
  // that produces those bytes on `producer`; it may be empty), then the piece is copied once
  // `producer` has got that far. Returns when everything has arrived in `dst`.
  int to_host(void* dst, const void* src, size_t bytes, hipStream_t producer,
              const std::function<int(size_t, size_t)>& before_piece);

 private:
  struct Impl;
  explicit Stager(Impl* impl) : impl_(impl) {}
  Impl* impl_;
};

}  // namespace pskv
#endif  // PSKV_STAGER_H_
