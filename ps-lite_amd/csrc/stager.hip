// The ring of pinned pieces and the worker threads behind Stager (stager.h).
#include "stager.h"

#include <algorithm>
#include <condition_variable>
#include <cstring>
#include <deque>
#include <mutex>
#include <new>
#include <thread>

#include "host_common.h"

namespace pskv {

struct Stager::Impl {
  int device = 0;
  hipStream_t copy = nullptr;  // the stream of the copy commands (default priority)
  char* ring = nullptr;        // kSlots pieces of pinned memory
  hipEvent_t dma_done[kSlots];   // the copy command that last used the slot has finished
  hipEvent_t prod_done[kSlots];  // device -> host: the producer has written the slot's piece

  std::mutex op_mu;  // one transfer at a time: the host link is what they would share anyway

  // worker threads: plain memcpy between caller memory and the ring
  struct Job {
    void* dst;
    const void* src;
    size_t len;
    int slot;
  };
  std::mutex mu;
  std::condition_variable cv_job, cv_done;
  std::deque<Job> jobs;
  int pending[kSlots] = {0};  // parts of the slot's piece that workers still owe

  char* slot_ptr(int s) const { return ring + (size_t)s * kPiece; }

  void work() {
    for (;;) {
      Job j;
      {
        std::unique_lock<std::mutex> lk(mu);
        cv_job.wait(lk, [&] { return !jobs.empty(); });
        j = jobs.front();
        jobs.pop_front();
      }
      std::memcpy(j.dst, j.src, j.len);
      bool last;
      {
        std::lock_guard<std::mutex> lk(mu);
        last = --pending[j.slot] == 0;
      }
      if (last) cv_done.notify_all();
    }
  }
  // A piece is copied in kParts parts by as many workers: it is ready (or gone) in a quarter of
  // the time, which is what a transfer of a few dozen pieces waits for at its start and its end.
  void submit(void* dst, const void* src, size_t len, int slot) {
    const size_t part = ((len + kParts - 1) / kParts + 4095) & ~(size_t)4095;
    int n = 0;
    {
      std::lock_guard<std::mutex> lk(mu);
      for (size_t at = 0; at < len; at += part, ++n)
        jobs.push_back(Job{static_cast<char*>(dst) + at, static_cast<const char*>(src) + at,
                           std::min(part, len - at), slot});
      pending[slot] = n;
    }
    if (n == 0) return;
    cv_job.notify_all();
  }
  void wait_slot(int slot) {
    std::unique_lock<std::mutex> lk(mu);
    cv_done.wait(lk, [&] { return pending[slot] == 0; });
  }
  bool slot_free(int slot) {
    std::lock_guard<std::mutex> lk(mu);
    return pending[slot] == 0;
  }
};

Stager* Stager::get(int device) {
  constexpr int kMaxDevices = 64;
  static std::mutex* mu = new std::mutex();
  static Stager* table[kMaxDevices] = {nullptr};
  static bool failed[kMaxDevices] = {false};
  if (device < 0 || device >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lk(*mu);
  if (table[device] || failed[device]) return table[device];
  // never destroyed: worker threads and pinned memory live until the process ends
  Impl* im = new (std::nothrow) Impl();
  if (!im) return nullptr;
  im->device = device;
  bool ok = hipStreamCreateWithFlags(&im->copy, hipStreamNonBlocking) == hipSuccess;
  ok = ok && hipHostMalloc(reinterpret_cast<void**>(&im->ring), (size_t)kSlots * kPiece, hipHostMallocDefault) ==
                 hipSuccess;
  for (int s = 0; ok && s < kSlots; ++s) {
    ok = hipEventCreateWithFlags(&im->dma_done[s], hipEventDisableTiming) == hipSuccess &&
         hipEventCreateWithFlags(&im->prod_done[s], hipEventDisableTiming) == hipSuccess;
  }
  if (!ok) {
    (void)hipGetLastError();
    failed[device] = true;  // (what was created stays; this happens once)
    return nullptr;
  }
  for (int w = 0; w < kWorkers; ++w) std::thread([im] { im->work(); }).detach();
  table[device] = new Stager(im);
  return table[device];
}

int Stager::to_device(void* dst, const void* src, size_t bytes, hipStream_t consumer,
                      const std::function<int(size_t, size_t)>& after_piece) {
  Impl* im = impl_;
  std::lock_guard<std::mutex> op(im->op_mu);
  const size_t npieces = (bytes + kPiece - 1) / kPiece;
  auto len_of = [&](size_t c) { return c + 1 < npieces ? kPiece : bytes - c * kPiece; };
  size_t issued = 0, sent = 0;
  int status = PSKV_OK;
  auto check = [&](hipError_t e) {
    if (e != hipSuccess && !status)
      status = set_error(PSKV_EHIP, "staging a request failed: %s", hipGetErrorString(e));
    return e == hipSuccess;
  };
  while (sent < npieces && status == PSKV_OK) {
    // keep the workers busy: the free slots of the ring get the next pieces. kSlack slots stay
    // behind the piece being sent, so that the wait below is for a copy command two or three
    // back and the copy engine always has the next command queued.
    while (issued < npieces && issued + kSlack < sent + kSlots) {
      const int slot = (int)(issued % kSlots);
      // the copy command that last read this slot (this transfer's or an earlier one's) is done
      if (!check(hipEventSynchronize(im->dma_done[slot]))) break;
      im->submit(im->slot_ptr(slot), static_cast<const char*>(src) + issued * kPiece, len_of(issued), slot);
      ++issued;
    }
    if (status) break;
    const int slot = (int)(sent % kSlots);
    const size_t off = sent * kPiece, len = len_of(sent);
    im->wait_slot(slot);
    if (!check(hipMemcpyAsync(static_cast<char*>(dst) + off, im->slot_ptr(slot), len, hipMemcpyHostToDevice,
                              im->copy)) ||
        !check(hipEventRecord(im->dma_done[slot], im->copy)) ||
        !check(hipStreamWaitEvent(consumer, im->dma_done[slot], 0)))
      break;
    if (after_piece) status = after_piece(off, len);
    ++sent;
  }
  if (status) {
    // the workers still read the caller's memory: it is the caller's again only when they are done
    for (int s = 0; s < kSlots; ++s) im->wait_slot(s);
  }
  return status;
}

int Stager::to_host(void* dst, const void* src, size_t bytes, hipStream_t producer,
                    const std::function<int(size_t, size_t)>& before_piece) {
  Impl* im = impl_;
  std::lock_guard<std::mutex> op(im->op_mu);
  const size_t npieces = (bytes + kPiece - 1) / kPiece;
  auto len_of = [&](size_t c) { return c + 1 < npieces ? kPiece : bytes - c * kPiece; };
  size_t launched = 0, drained = 0;
  int status = PSKV_OK;
  while (drained < npieces && status == PSKV_OK) {
    // Produce and send off every piece whose slot is free (the worker that emptied it for an
    // earlier piece is done); never wait for a worker while pieces that have arrived could be
    // handed to the others.
    while (launched < npieces && launched < drained + kSlots) {
      const int slot = (int)(launched % kSlots);
      if (!im->slot_free(slot)) {
        if (drained < launched) break;  // hand out what has arrived first
        im->wait_slot(slot);
      }
      const size_t off = launched * kPiece, len = len_of(launched);
      if (before_piece) {
        status = before_piece(off, len);
        if (status) break;
      }
      hipError_t e = hipEventRecord(im->prod_done[slot], producer);
      if (e == hipSuccess) e = hipStreamWaitEvent(im->copy, im->prod_done[slot], 0);
      if (e == hipSuccess)
        e = hipMemcpyAsync(im->slot_ptr(slot), static_cast<const char*>(src) + off, len, hipMemcpyDeviceToHost,
                           im->copy);
      if (e == hipSuccess) e = hipEventRecord(im->dma_done[slot], im->copy);
      if (e != hipSuccess) {
        status = set_error(PSKV_EHIP, "staging a response failed: %s", hipGetErrorString(e));
        break;
      }
      ++launched;
    }
    if (status) break;
    const int slot = (int)(drained % kSlots);
    const hipError_t e = hipEventSynchronize(im->dma_done[slot]);
    if (e != hipSuccess) {
      status = set_error(PSKV_EHIP, "staging a response failed: %s", hipGetErrorString(e));
      break;
    }
    im->submit(static_cast<char*>(dst) + drained * kPiece, im->slot_ptr(slot), len_of(drained), slot);
    ++drained;
  }
  // nothing of this transfer may be left in the ring or in flight when the caller gets its buffer
  for (int s = 0; s < kSlots; ++s) im->wait_slot(s);
  if (status) (void)hipStreamSynchronize(im->copy);
  return status;
}

}  // namespace pskv
