// Host side of the HBM-resident key-value store: owns the slot array, the row
// arena and the per-request workspace, sizes them, and enqueues the kernels of
// table_kernels.h in request order on one stream. This is what a ps-lite server
// calls in place of KVServerDefaultHandle (include/ps/kv_app.h:440-463).
#include <algorithm>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <memory>
#include <mutex>
#include <new>
#include <string>
#include <thread>
#include <vector>

#include <hip/hip_ext.h>

#include "host_common.h"
#include "scan.h"
#include "stager.h"
#include "table_kernels.h"

namespace pskv {

static thread_local std::string g_last_error;

int set_error(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}
void clear_error() { g_last_error.clear(); }

namespace {

constexpr uint64_t kDefaultCapacity = 1u << 20;
constexpr uint64_t kMinSlots = 1024;
constexpr unsigned kMaxGrid = 1u << 20;
// The write-back of the SCALAR key cache mostly finds nothing to do (the request in flight repeats
// the cached keys, or the slots are up to date), and a launch costs by the workgroup even then:
// 62,500 workgroups that leave at once took 15 us. It strides over the keys with this many.
constexpr unsigned kFlushGrid = 4096;
constexpr size_t kMaxProfSamples = 65536;
constexpr uint64_t kSlackBytes = 256ull << 20;  // tables up to this size trade memory for fewer waits
// A slot array that could run short is replaced without asking the device first while the larger
// one stays below this size; beyond it the host waits for exact counters before it spends the memory.
constexpr uint64_t kGrowUnaskedBytes = 4096ull << 20;
constexpr uint64_t kKeepInFlight = 2;  // requests the host leaves unaccounted for when it lets the device catch up
// ... unless the array that the uncertainty would cost is this large: then it lets the device catch up all the way
constexpr uint64_t kLargeArrayBytes = 1024ull << 20;
constexpr uint64_t kSpareMaxBytes = 16384ull << 20;  // no array larger than this is allocated ahead of need
// Host-resident requests up to this size (per direction) skip the copy commands: the kernels
// read the request from, and write the response to, pinned host memory mapped into the GPU.
constexpr size_t kSmallBytes = 1024u << 10;
constexpr int kSmallParts = 8;  // (128 KiB each: a SCALAR push of up to 10,000 keys)
// Host-resident buffers from this size on travel piece by piece through the ring of pinned memory
// (stager.h), copying, transfer and kernels overlapping; smaller ones take one copy command.
constexpr size_t kPipeBytes = 4u << 20;
// The fill a slot array never exceeds, whatever the host assumed about the requests in flight (reserve()).
constexpr double kHardLoad = 0.85;

// A device buffer that only grows. Contents are not kept across growth.
struct GrowBuf {
  void* ptr = nullptr;
  size_t bytes = 0;
};

struct EventPair {
  hipEvent_t a, b;
};

// An allocation handed to the library's allocating thread (AllocWorker below).
struct AllocJob {
  int device = 0;
  size_t bytes = 0;
  hipStream_t stream = nullptr;
  void* ptr = nullptr;
  bool pooled = false;
  int rc = PSKV_OK;
  double took_us = 0;  // what the allocation cost the allocating thread
  bool done = false;  // guarded by AllocWorker::mu
};


// What the host reads back of the device state, written by the device into pinned host memory
// (a one-wavefront kernel is quicker than a copy command for these few words).
struct StateView {
  uint64_t count;       // keys held, the side slot included
  uint64_t arena_top;
  uint64_t scan_total;
  uint64_t same_epoch;
  unsigned error, req_error, special_present, pad;
};

// One wavefront per table (blockIdx.x).
struct StateBatch {
  const DevState* st[kMaxBatch];
  StateView* out[kMaxBatch];
};
__global__ void k_read_state(StateBatch sb) {
  const DevState* st = sb.st[blockIdx.x];
  StateView* out = sb.out[blockIdx.x];
  unsigned long long c = threadIdx.x < kCountShards ? st->count_shard[threadIdx.x * kShardStride] : 0ull;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o);
  if (threadIdx.x != 0) return;
  out->count = c;
  out->arena_top = st->arena_top;
  out->scan_total = st->scan_total;
  out->same_epoch = st->same_epoch;
  out->error = st->error;
  out->req_error = st->req_error;
  out->special_present = st->special_present;
}

}  // namespace
}  // namespace pskv

using namespace pskv;

struct pskv_table {
  int device = 0;
  int mode = PSKV_MODE_SCALAR;
  hipStream_t stream = nullptr;
  bool own_stream = false;
  float max_load = 0.5f;

  Slot* slots = nullptr;
  bool slots_pooled = false, arena_pooled = false;  // taken from the stream-ordered pool by a growth
  uint64_t cap = 0;        // slots, a power of two
  // The array the next growth will move into, allocated ahead of need (once the table is 40 % of
  // the way to that growth) at the end of a request, while the GPU is busy with that request:
  // allocating costs the host 50-100 us, which would otherwise be spent with the GPU idle.
  Slot* spare = nullptr;
  uint64_t spare_cap = 0;
  bool spare_pooled = false;
  std::shared_ptr<AllocJob> spare_job;  // the allocation of `spare` while it is under way
  // what the sizing logic did, printed when the table goes if PSKV_STATS is set in the environment
  struct Stats {
    uint64_t requests = 0, waits = 0, growths = 0, growths_unasked = 0, spare_used = 0, records = 0, catch_ups = 0;
    double alloc_us = 0, release_us = 0, catch_up_us = 0;  // host time spent allocating, releasing, catching up
    double ahead_us = 0;  // time the allocating thread spent on this table's arrays
  } stats;
  uint64_t count = 0;      // key count at the last read_state()

  // Host-side bounds of what the device counters can have reached. Requests are enqueued
  // without waiting, so the host only knows exact counters (`base_*`) as of request
  // `base_seq` and must assume that every key of a later request was new (`pend_*`).
  // A published snapshot (below) moves the base forward without a stream wait.
  uint64_t seq = 0;        // requests begun so far
  uint64_t base_seq = 0;   // base_count / base_top hold after all requests < base_seq
  uint64_t base_count = 0, base_top = 0;
  uint64_t pend_keys = 0, pend_units = 0;  // sums of the log over [base_seq, seq)
  static const int kLog = 64;
  uint64_t log_keys[kLog] = {0}, log_units[kLog] = {0};
  Snapshot* snap = nullptr;  // pinned host memory the device publishes into
  uint64_t record_seq = ~0ull;  // the newest request that was asked to publish its counters (all ones: none yet)
  double new_share = 0.0;  // share of the keys named by requests that were new, over the latest records
  bool share_known = false;  // (a record has said so)
  DevState* st = nullptr;  // device
  StateView* st_host = nullptr;  // pinned: what read_state() last read of the device state

  // row modes
  float* arena = nullptr;
  uint64_t arena_cap = 0;  // floats
  uint64_t row_len = 0;    // FIXED

  GrowBuf ws;         // per-request workspace (row references, offsets)
  GrowBuf tiles;      // VARLEN: first key of every request-side tile
  GrowBuf tiles_aff;  // VARLEN: one TileNote per tile
  char* small_in = nullptr;   // pinned, kSmallBytes: small host-resident requests, read in place
  char* small_out = nullptr;  // pinned, kSmallBytes: their responses, written in place
  // A small host-resident SCALAR push returns once its kernel is queued: nothing comes back from
  // it. Such pushes take the kSmallParts parts of small_in in turn (when they fit one), so that
  // several can be in flight; a request that writes a part waits for the event its last user left.
  hipEvent_t small_done[kSmallParts] = {nullptr};
  bool small_pending[kSmallParts] = {false};
  int small_next = 0;      // the part the next such push takes
  int small_newest = -1;   // the part whose event was recorded last (everything before it is done when it is)
  GrowBuf stage;      // device copies of host-resident request buffers
  GrowBuf stage_out;  // device-side response of a host-resident or undersized pull
  bool no_growth = false;  // set while dumping: every key is known to be present
  // Recorded requests (pskv_replay_*): `gen` counts the requests that went the ordinary way, each
  // of which may move a buffer, refill the key cache or write cached values back, so a recording
  // only runs while `gen` is what it was when the recording was made. `capturing`: the table's
  // stream is being captured into a HIP graph, nothing may be allocated, waited for or timed.
  uint64_t gen = 0;
  bool capturing = false;

  // Row modes: the workspace keeps the row references, offsets and tile table of the last
  // request that computed them, and the key cache keeps that request's keys and lens, so a
  // request with the same keys (the usual case for a parameter server) can skip the lens
  // scan and every hash probe. The device decides whether the keys match; these fields only
  // say whether the buffers still have the shape the cached request gave them.
  GrowBuf cache_keys, cache_lens;
  bool cache_valid = false;
  uint64_t cache_n = 0, cache_nvals = 0;
  uint64_t epoch = 0;  // number of the last request that took part in this

  // SCALAR: the same idea with the VALUES of the cached keys kept in request order (and the
  // slot number of every key), so that a request which repeats the cached key set streams
  // through `sc_vals` and touches no slot; the slots are brought up to date before anything
  // else reads or changes them (`sc_dirty`: they may be behind).
  GrowBuf sc_vals, sc_slots;
  bool sc_dirty = false;
  uint64_t sc_last_n = 0;   // keys of the previous request: a size that repeats is worth recording
  int sc_last_kind = -1;    // and its kind (0: push or push+pull, 1: pull)
  unsigned sc_pairs = 0;    // pulls in a row (up to 2) that came right behind a push of their own size
  // What the comparisons of the two kinds of requests (0: pushes and push+pulls, 1: pulls) have
  // come to lately: pushes that bring new keys every time may still leave a cache behind that the
  // pull after each of them is served from.
  struct ScTrack {
    unsigned fail = 0;  // comparisons in a row that found other keys
    unsigned skip = 0;  // requests of this kind left to run without a comparison after such failures
    bool hit = false;   // the newest comparison of this kind found the cached keys
  } sc_track[2];
  static const int kScKinds = 64;
  unsigned char sc_kind[kScKinds] = {0};  // kind of the request with number e, at e % kScKinds
  unsigned long long* outcome = nullptr;  // pinned: epoch << 1 | same of the newest comparison
  unsigned long long sc_seen = 0;         // the value of *outcome the host last looked at
  uint64_t sc_min_keys = 0;               // requests below this size leave the cache alone; 0 = no cache

  bool counted = false;  // among the live tables of its device
  bool prof = false;
  std::vector<EventPair> pending[PSKV_KERNEL_COUNT];
  std::vector<EventPair> free_events;
  uint64_t launches[PSKV_KERNEL_COUNT] = {0};
  double total_ms[PSKV_KERNEL_COUNT] = {0};
  std::vector<float> samples[PSKV_KERNEL_COUNT];  // per-launch durations, bounded
};

namespace {

// ---- profiling -------------------------------------------------------------------
// Launches `kernel` on the table's stream. While profiling is on, the launch carries
// a start and a stop event of its own (hipExtLaunchKernelGGL), which take the
// begin/end timestamps of that very dispatch: the same clock a profiler reads,
// without the idle time that events recorded around a launch would add.
template <typename... KArgs, typename... Args>
void launch_lds(pskv_table* t, int prof_kernel, void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds,
                Args... args) {
  if (t->prof && prof_kernel >= 0 && !t->capturing) {
    EventPair ev;
    bool have = false;
    if (!t->free_events.empty()) {
      ev = t->free_events.back();
      t->free_events.pop_back();
      have = true;
    } else if (hipEventCreate(&ev.a) == hipSuccess) {
      if (hipEventCreate(&ev.b) == hipSuccess) {
        have = true;
      } else {
        (void)hipEventDestroy(ev.a);
      }
    }
    if (have) {
      hipExtLaunchKernelGGL(kernel, grid, block, lds, t->stream, ev.a, ev.b, 0, static_cast<KArgs>(args)...);
      t->pending[prof_kernel].push_back(ev);
      return;
    }
  }
  hipLaunchKernelGGL(kernel, grid, block, lds, t->stream, static_cast<KArgs>(args)...);
}

template <typename... KArgs, typename... Args>
void launch(pskv_table* t, int prof_kernel, void (*kernel)(KArgs...), dim3 grid, dim3 block,
            Args... args) {
  launch_lds(t, prof_kernel, kernel, grid, block, 0, args...);
}

int prof_collect(pskv_table* t) {
  PSKV_HIP(hipStreamSynchronize(t->stream));
  for (int k = 0; k < PSKV_KERNEL_COUNT; ++k) {
    for (const EventPair& ev : t->pending[k]) {
      float ms = 0.f;
      if (hipEventElapsedTime(&ms, ev.a, ev.b) == hipSuccess) {
        t->total_ms[k] += ms;
        t->launches[k] += 1;
        if (t->samples[k].size() < kMaxProfSamples) t->samples[k].push_back(ms);
      }
      t->free_events.push_back(ev);
    }
    t->pending[k].clear();
  }
  return PSKV_OK;
}

// ---- memory ----------------------------------------------------------------------
int grow(pskv_table* t, GrowBuf* b, size_t bytes) {
  if (bytes <= b->bytes) return PSKV_OK;
  if (t->capturing) return set_error(PSKV_ESTALE, "a recorded request needs a buffer that its first run did not leave");
  // An eighth to spare (up to 32 MB): the slices of a worker's requests differ by a few keys from one
  // request to the next, and a reallocation waits for the stream and costs 100-350 us, several
  // requests' worth, every time a table sees its largest slice so far.
  size_t want = std::max(bytes + std::min<size_t>(bytes / 8, (size_t)32 << 20), b->bytes + b->bytes / 2);
  want = (want + 4095) & ~(size_t)4095;
  if (b == &t->ws || b == &t->tiles || b == &t->tiles_aff || b == &t->cache_keys ||
      b == &t->cache_lens || b == &t->sc_vals || b == &t->sc_slots)
    t->cache_valid = false;  // the contents do not survive a reallocation
  if (b->ptr) {
    // earlier requests on the stream may still read the old buffer
    PSKV_HIP(hipStreamSynchronize(t->stream));
    PSKV_HIP(hipFree(b->ptr));
    b->ptr = nullptr;
    b->bytes = 0;
  }
  PSKV_HIP(hipMalloc(&b->ptr, want));
  b->bytes = want;
  return PSKV_OK;
}

// Carves aligned pieces out of a GrowBuf that was grown to the total beforehand.
struct Carver {
  char* base;
  size_t at = 0;
  explicit Carver(void* p) : base(static_cast<char*>(p)) {}
  template <typename T>
  T* take(size_t count) {
    T* r = reinterpret_cast<T*>(base + at);
    at += (count * sizeof(T) + 255) & ~(size_t)255;
    return r;
  }
  static size_t need(size_t count, size_t elem) { return (count * elem + 255) & ~(size_t)255; }
};

// What the host keeps of a state that k_read_state has just written (the stream is idle).
void adopt_state(pskv_table* t) {
  const uint64_t c = t->st_host->count;
  t->count = c;
  // everything enqueued so far is complete: the bounds become exact
  t->base_seq = t->seq;
  t->base_count = c;
  t->base_top = t->st_host->arena_top;
  t->pend_keys = t->pend_units = 0;
}

int read_state(pskv_table* t) {
  StateBatch sb;
  std::memset(&sb, 0, sizeof(sb));
  sb.st[0] = t->st;
  sb.out[0] = t->st_host;
  k_read_state<<<dim3(1), dim3(64), 0, t->stream>>>(sb);
  PSKV_HIP(hipGetLastError());
  PSKV_HIP(hipStreamSynchronize(t->stream));
  adopt_state(t);
  return PSKV_OK;
}

// Turns device error bits into a status, clearing them on the device.
int report_device_errors(pskv_table* t) {
  const unsigned bits = t->st_host->error | t->st_host->req_error;
  if (!bits) return PSKV_OK;
  PSKV_HIP(hipMemsetAsync(&t->st->error, 0, 2 * sizeof(unsigned), t->stream));
  PSKV_HIP(hipStreamSynchronize(t->stream));
  if (bits & kDevErrFull) return set_error(PSKV_ENOMEM, "slot array full (internal sizing error)");
  if (bits & kDevErrReplay)
    return set_error(PSKV_ESTALE, "a replayed request no longer named the keys it was recorded with: that run of it "
                                  "changed and answered nothing on this table");
  if (bits & kDevErrBadLen)
    return set_error(PSKV_EINVAL, "a length is negative or above PSKV_MAX_VARLEN_ROW");
  if (bits & kDevErrSizeMismatch)
    return set_error(PSKV_ESIZE_MISMATCH, "lens do not add up to the number of values");
  if (bits & kDevErrDuplicate)
    return set_error(PSKV_EINVAL, "a request held the same key twice (keys must be unique)");
  if (bits & kDevErrNoRoom)
    return set_error(PSKV_ESIZE_MISMATCH, "a var-len pull response did not fit the caller's buffer");
  return set_error(PSKV_ELEN_CHANGED, "a pushed row length differs from the stored length");
}

// Slot arrays and arenas come from, and go back to, the device's stream-ordered pool where the
// runtime has one (PSKV_NO_ASYNC_ALLOC in the environment goes back to hipMalloc / hipFree): a
// growth releases the old array behind the kernel that empties it, without a wait on the host
// (a plain hipFree of a few hundred MB blocks the host for 150-440 us, longer than the
// re-insertion itself). `pooled` says how the array must be released later.
// The pool is the library's own, one per device, and keeps what is freed into it: the default
// pool hands freed memory back to the system at the next wait of any stream, which for the old
// array of a growth is an unmapping of hundreds of microseconds in the middle of the caller's
// loop. pskv_device_trim gives the kept memory back; so does the end of the last table.
struct DevicePool {
  std::atomic<int> known{0};  // 0 = not asked yet, 1 = no pool, 2 = pool
  hipMemPool_t pool = nullptr;
  std::atomic<long> tables{0};  // live tables on the device
};
DevicePool g_pools[64];

hipMemPool_t device_pool(int dev) {
  if (dev < 0 || dev >= 64) return nullptr;
  DevicePool& dp = g_pools[dev];
  int k = dp.known.load(std::memory_order_acquire);
  if (k == 0) {
    static std::mutex mu;
    std::lock_guard<std::mutex> lock(mu);
    k = dp.known.load(std::memory_order_acquire);
    if (k == 0) {
      int ok = 0;
      if (std::getenv("PSKV_NO_ASYNC_ALLOC") ||
          hipDeviceGetAttribute(&ok, hipDeviceAttributeMemoryPoolsSupported, dev) != hipSuccess)
        ok = 0;
      if (ok) {
        hipMemPoolProps props;
        std::memset(&props, 0, sizeof(props));
        props.allocType = hipMemAllocationTypePinned;
        props.handleTypes = hipMemHandleTypeNone;
        props.location.type = hipMemLocationTypeDevice;
        props.location.id = dev;
        uint64_t keep = ~0ull;
        if (hipMemPoolCreate(&dp.pool, &props) != hipSuccess ||
            hipMemPoolSetAttribute(dp.pool, hipMemPoolAttrReleaseThreshold, &keep) != hipSuccess) {
          dp.pool = nullptr;
          ok = 0;
        }
      }
      (void)hipGetLastError();
      k = ok ? 2 : 1;
      dp.known.store(k, std::memory_order_release);
    }
  }
  return k == 2 ? dp.pool : nullptr;
}

int alloc_for_growth(void** out, size_t bytes, hipStream_t stream, bool* pooled) {
  int dev = 0;
  hipMemPool_t pool = hipGetDevice(&dev) == hipSuccess ? device_pool(dev) : nullptr;
  if (pool) {
    if (hipMallocFromPoolAsync(out, bytes, pool, stream) == hipSuccess) {
      *pooled = true;
      return PSKV_OK;
    }
    (void)hipGetLastError();
  }
  *pooled = false;
  PSKV_HIP(hipMalloc(out, bytes));
  return PSKV_OK;
}

// Allocating a few hundred MB costs the calling thread 50 us on a good day and 800 on a bad one,
// so the array of a coming growth is allocated by a thread of the library's own while the
// caller goes on enqueuing requests; the growth picks the result up (and waits for it in the
// unlikely case that it is not there yet). One thread per process, started with the first job,
// kept until the process ends.
class AllocWorker {
 public:
  static AllocWorker& get() {
    static AllocWorker* w = new AllocWorker();  // never destroyed: its thread may outlive static destructors
    return *w;
  }
  void submit(const std::shared_ptr<AllocJob>& job) {
    {
      std::lock_guard<std::mutex> lk(mu_);
      if (!started_) {
        std::thread(&AllocWorker::run, this).detach();
        started_ = true;
      }
      jobs_.push_back(job);
    }
    cv_job_.notify_one();
  }
  void wait(const std::shared_ptr<AllocJob>& job) {
    std::unique_lock<std::mutex> lk(mu_);
    cv_done_.wait(lk, [&] { return job->done; });
  }
  bool finished(const std::shared_ptr<AllocJob>& job) {
    std::lock_guard<std::mutex> lk(mu_);
    return job->done;
  }

 private:
  void run() {
    for (;;) {
      std::shared_ptr<AllocJob> job;
      {
        std::unique_lock<std::mutex> lk(mu_);
        cv_job_.wait(lk, [&] { return !jobs_.empty(); });
        job = jobs_.front();
        jobs_.pop_front();
      }
      const auto a0 = std::chrono::steady_clock::now();
      if (hipSetDevice(job->device) != hipSuccess) {
        (void)hipGetLastError();
        job->rc = PSKV_EHIP;
      } else {
        job->rc = alloc_for_growth(&job->ptr, job->bytes, job->stream, &job->pooled);
      }
      job->took_us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - a0).count();
      {
        std::lock_guard<std::mutex> lk(mu_);
        job->done = true;
      }
      cv_done_.notify_all();
    }
  }
  std::mutex mu_;
  std::condition_variable cv_job_, cv_done_;
  std::deque<std::shared_ptr<AllocJob>> jobs_;
  bool started_ = false;
};

// Releases an array that kernels already enqueued on `stream` may still use.
int release_after(void* ptr, bool pooled, hipStream_t stream) {
  if (!ptr) return PSKV_OK;
  if (pooled) {
    PSKV_HIP(hipFreeAsync(ptr, stream));
    return PSKV_OK;
  }
  PSKV_HIP(hipStreamSynchronize(stream));
  PSKV_HIP(hipFree(ptr));
  return PSKV_OK;
}

int alloc_slots(uint64_t cap, Slot** out, hipStream_t stream, bool* pooled, bool fill = true) {
  int rc = alloc_for_growth(reinterpret_cast<void**>(out), cap * sizeof(Slot), stream, pooled);
  if (rc) return rc;
  // all-ones bytes: key = empty marker (k_regrow writes every slot itself and needs no fill)
  if (fill) PSKV_HIP(hipMemsetAsync(*out, 0xFF, cap * sizeof(Slot), stream));
  return PSKV_OK;
}

// Moves the base of the bounds forward to the newest record the device has published: the
// counters after request `seq_end`.
void adopt_snapshot(pskv_table* t) {
  const Snapshot* sn = t->snap;
  const uint64_t s1 = sn->seq_end;
  std::atomic_thread_fence(std::memory_order_acquire);
  const uint64_t c = sn->count, top = sn->arena_top;
  std::atomic_thread_fence(std::memory_order_acquire);
  const uint64_t s0 = sn->seq_begin;
  if (s0 != s1 || s1 < t->base_seq || s1 >= t->seq) return;  // (the initial record is all ones)
  uint64_t named = 0;
  for (uint64_t r = t->base_seq; r <= s1; ++r) {
    named += t->log_keys[r % pskv_table::kLog];
    t->pend_keys -= t->log_keys[r % pskv_table::kLog];
    t->pend_units -= t->log_units[r % pskv_table::kLog];
  }
  // which share of the keys that requests named turned out to be new, lately (a moving average)
  if (named) {
    const double share = c > t->base_count ? std::min(1.0, (double)(c - t->base_count) / (double)named) : 0.0;
    t->new_share = t->share_known ? 0.5 * t->new_share + 0.5 * share : share;
    t->share_known = true;
  }
  t->base_seq = s1 + 1;
  t->base_count = c;
  t->base_top = top;
}

// SCALAR: brings the slots up to date with the values of the key cache. Enqueued before
// anything but the kernels of a request that repeats the cached keys looks at the slots.
int flush_scalar_cache(pskv_table* t) {
  if (!t->sc_dirty) return PSKV_OK;
  ReqBatch rb;
  std::memset(&rb, 0, sizeof(rb));
  TableReq& d = rb.t[0];
  d.slots = t->slots;
  d.mask = t->cap - 1;
  d.st = t->st;
  d.n = t->cache_n;
  d.arena = static_cast<float*>(t->sc_vals.ptr);
  d.tile_key = static_cast<uint32_t*>(t->sc_slots.ptr);
  d.cache_mode = kFlushAlways;
  d.nblk = grid_for(t->cache_n, kBlock, kFlushGrid);
  hipLaunchKernelGGL(k_scalar_flush, dim3(d.nblk, 1), dim3(kBlock), 0, t->stream, rb);
  PSKV_HIP(hipGetLastError());
  t->sc_dirty = false;
  return PSKV_OK;
}

// Takes over the array that the allocating thread was asked for, if it is there (`wait`: or
// once it is there).
void collect_spare(pskv_table* t, bool wait) {
  if (!t->spare_job) return;
  if (wait) {
    const auto w0 = std::chrono::steady_clock::now();
    AllocWorker::get().wait(t->spare_job);
    t->stats.alloc_us += std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - w0).count();
  } else if (!AllocWorker::get().finished(t->spare_job)) {
    return;
  }
  t->stats.ahead_us += t->spare_job->took_us;
  if (t->spare_job->rc == PSKV_OK && t->spare_job->ptr) {
    t->spare = static_cast<Slot*>(t->spare_job->ptr);
    t->spare_pooled = t->spare_job->pooled;
  } else {
    t->spare_cap = 0;  // (the growth will ask again itself and report)
  }
  t->spare_job.reset();
}

// The slots a growth goes to when the table has to hold `keys_needed` keys: at least twice the
// slots; four times while that stays a small array (a table that starts at the default size and
// keeps growing then moves its keys half as often on the way up).
uint64_t grown_cap(const pskv_table* t, uint64_t keys_needed) {
  const uint64_t want = next_pow2((uint64_t)((double)keys_needed / t->max_load) + 1);
  return std::max(want, t->cap * 4 * sizeof(Slot) <= kSlackBytes ? t->cap * 4 : t->cap * 2);
}

int grow_slots(pskv_table* t, uint64_t keys_needed) {
  uint64_t want = grown_cap(t, keys_needed);
  Slot* fresh = nullptr;
  int rc = PSKV_OK;
  if (t->mode == PSKV_MODE_SCALAR) {
    // the key cache holds slot numbers of the old array, and values the old array may lack
    rc = flush_scalar_cache(t);
    if (rc) return rc;
    t->cache_valid = false;
  }
  bool pooled = false;
  ++t->stats.growths;
  collect_spare(t, true);
  if (t->spare && t->spare_cap >= want) {
    ++t->stats.spare_used;
    fresh = t->spare;
    want = t->spare_cap;
    pooled = t->spare_pooled;
  } else {
    if (t->spare) {  // too small after all
      rc = release_after(t->spare, t->spare_pooled, t->stream);
      if (rc) return rc;
    }
    const auto a0 = std::chrono::steady_clock::now();
    rc = alloc_slots(want, &fresh, t->stream, &pooled, false);
    t->stats.alloc_us += std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - a0).count();
    if (rc) return rc;
  }
  t->spare = nullptr;
  t->spare_cap = 0;
  const uint64_t factor = want / t->cap;
  if (factor <= (uint64_t)kRegrowMaxFactor) {
    // two streaming passes: the new array is written whole, slot by slot, from LDS
    const unsigned nblk = (unsigned)(t->cap / kRegrowOld);
    const size_t lds = (size_t)kRegrowOld * factor * 2 * sizeof(unsigned long long);
    launch_lds(t, PSKV_KERNEL_REHASH, k_regrow, dim3(nblk), dim3(kBlock), lds, t->slots, fresh, t->cap - 1,
               want - 1, (unsigned)factor);
    PSKV_HIP(hipGetLastError());
    launch(t, PSKV_KERNEL_REHASH, k_regrow_rest, dim3((nblk * kRestLanes + kBlock - 1) / kBlock), dim3(kBlock),
           (const Slot*)t->slots, t->cap, fresh, want - 1, t->st);
  } else {
    // (a small table that a large request makes much larger: fill and scatter)
    PSKV_HIP(hipMemsetAsync(fresh, 0xFF, want * sizeof(Slot), t->stream));
    launch(t, PSKV_KERNEL_REHASH, k_rehash, dim3(grid_for(t->cap, kBlock, kMaxGrid)), dim3(kBlock),
           (const Slot*)t->slots, t->cap, fresh, want - 1, t->st);
  }
  PSKV_HIP(hipGetLastError());
  const auto r0 = std::chrono::steady_clock::now();
  rc = release_after(t->slots, t->slots_pooled, t->stream);
  t->stats.release_us += std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - r0).count();
  t->slots = fresh;
  t->slots_pooled = pooled;
  t->cap = want;
  return rc;
}

// Called at the end of a request, with its kernels queued: allocates the array of the next growth
// once the keys the table is known to hold have come 40 % of the way to that growth.
void prepare_growth(pskv_table* t) {
  if (t->spare || t->spare_job || t->no_growth) return;
  adopt_snapshot(t);  // (a read of pinned memory)
  const double limit = (double)t->max_load * (double)t->cap;
  // the keys known to be held, plus, while requests have mostly been bringing new keys, the share of
  // the keys in flight that will be new if that goes on (a caller that runs far ahead of the device
  // would otherwise learn too late how full the table is)
  const double expected = (double)t->base_count + (t->new_share >= 0.5 ? t->new_share * (double)t->pend_keys : 0.0);
  if (expected <= 0.4 * limit) return;
  const uint64_t want = grown_cap(t, 0);
  if (want * sizeof(Slot) > kSpareMaxBytes) return;
  std::shared_ptr<AllocJob> job = std::make_shared<AllocJob>();
  job->device = t->device;
  job->bytes = want * sizeof(Slot);
  job->stream = t->stream;
  t->spare_cap = want;
  t->spare_job = job;
  AllocWorker::get().submit(job);
}

int grow_arena(pskv_table* t, uint64_t floats_needed, uint64_t live_floats) {
  uint64_t want = std::max(floats_needed, t->arena_cap + t->arena_cap / 2);
  want = (want + 1023) & ~(uint64_t)1023;
  float* fresh = nullptr;
  bool pooled = false;
  int rc = alloc_for_growth(reinterpret_cast<void**>(&fresh), want * sizeof(float), t->stream, &pooled);
  if (rc) return rc;
  if (live_floats && t->arena) {
    PSKV_HIP(hipMemcpyAsync(fresh, t->arena, live_floats * sizeof(float), hipMemcpyDeviceToDevice,
                            t->stream));
  }
  rc = release_after(t->arena, t->arena_pooled, t->stream);
  t->arena = fresh;
  t->arena_pooled = pooled;
  t->arena_cap = want;
  return rc;
}

// Begins a request that may create up to `n` keys and take up to `units` allocation units
// of the arena (rows for FIXED, 16 bytes for VARLEN; `floats_per_unit` converts to floats).
// Grows the slot array / the arena first if the bounds say they could overflow. The fast
// path touches no device state; the next best reads the snapshot the device published;
// only then does it wait for the stream and read the counters.
//
// Close to a limit the device publishes its counters as they are after the request, so that a
// later request can move the base forward without waiting for the stream: `pub->snap` is
// set when a record is wanted, and the caller hands it to the kernel of the request that
// changes the counters.
struct PublishReq {
  Snapshot* snap = nullptr;
  uint64_t seq = 0;
};

int reserve(pskv_table* t, uint64_t n, uint64_t units, uint64_t floats_per_unit, PublishReq* pub) {
  if (t->no_growth) return PSKV_OK;
  // Two limits. `limit` is the fill the table is kept below; `hard` (0.85 unless max_load is higher) is
  // the fill it must never exceed. The keys in flight count in full against the second, and against the
  // first with the share of them that is going to be new if requests go on as the latest records say
  // (twice that share plus a tenth, to be on the safe side; in full while no record has said anything).
  // A server whose requests mostly name keys it holds, the steady state of a parameter server, then does
  // not grow, or wait, for keys that are not coming, however far ahead of the device its caller runs; if
  // the requests change their ways the table runs fuller than `limit` for as long as it takes the next
  // records to say so, never fuller than `hard`.
  const double limit = (double)t->max_load * (double)t->cap;
  const double hard = std::max((double)t->max_load, kHardLoad) * (double)t->cap;
  auto slots_short = [&]() {
    // (looked up on every call: a record adopted further down may have changed it)
    const double share = t->share_known ? std::min(1.0, 2.0 * t->new_share + 0.1) : 1.0;
    const double in_flight = (double)(t->pend_keys + n);
    return (double)t->base_count + in_flight > hard || (double)t->base_count + share * in_flight > limit;
  };
  auto arena_short = [&]() {
    return units && (t->base_top + t->pend_units + units) * floats_per_unit > t->arena_cap;
  };
  // an ageing base is refreshed from the newest record whenever one has arrived (a host read)
  if (t->seq - t->base_seq >= (uint64_t)pskv_table::kLog / 4) adopt_snapshot(t);
  if (slots_short() || arena_short() || t->seq - t->base_seq >= (uint64_t)pskv_table::kLog - 1) {
    adopt_snapshot(t);
    const bool old_log = t->seq - t->base_seq >= (uint64_t)pskv_table::kLog - 1;
    // (two requests of 16M keys that are left unaccounted for would make a 1 GiB array a 2 GiB one;
    // the host's lead is worth less than that: a few tens of microseconds of idle GPU, once)
    const uint64_t keep =
        grown_cap(t, t->base_count + t->pend_keys + n) * sizeof(Slot) >= kLargeArrayBytes ? 0 : kKeepInFlight;
    if (slots_short() && !arena_short() && !old_log && (double)(t->base_count + n) <= limit &&
        t->record_seq != ~0ull && t->record_seq >= t->base_seq && t->seq - t->base_seq > keep) {
      // The array is only short if the requests in flight create most of their keys, and some of
      // them are going to say how many they did create: the host lets the device catch up, but not
      // all the way (unless a large array is at stake). A caller that runs many requests ahead is held
      // back until only kKeepInFlight requests are unaccounted for (so the device never runs dry, as it would in a wait for the
      // stream, and the steps that follow do not run in lock-step with the host); if the array
      // still looks short then, it is replaced, at most that many requests early and sized for
      // at most that many requests of uncertainty.
      const auto t0 = std::chrono::steady_clock::now();
      unsigned spins = 0;
      while (slots_short() && (double)(t->base_count + n) <= limit && t->record_seq >= t->base_seq &&
             t->seq - t->base_seq > keep) {
        adopt_snapshot(t);
        if ((++spins & 63u) == 0) {
          if (std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(20)) break;
          std::this_thread::yield();
        }
      }
      ++t->stats.catch_ups;
      t->stats.catch_up_us += std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
    }
    if (slots_short() && !arena_short() && !old_log &&
        grown_cap(t, t->base_count + t->pend_keys + n) * sizeof(Slot) <= kGrowUnaskedBytes) {
      // Only the slots could run short, and the larger array is not a large one: it is taken now,
      // sized for what the requests in flight could create at most, without asking the device how
      // many keys they did create. The move is queued behind them; nothing waits.
      const uint64_t most = t->base_count + t->pend_keys + n;
      // (room for two more such requests while that keeps the array a small one)
      const uint64_t slack_n = grown_cap(t, most + 2 * n) * sizeof(Slot) <= kSlackBytes ? 2 * n : 0;
      int rc = grow_slots(t, most + slack_n);
      if (rc) return rc;
      ++t->stats.growths_unasked;
    } else if (slots_short() || arena_short() || old_log) {
      int rc = read_state(t);  // exact counters, stream idle
      if (rc) return rc;
      ++t->stats.waits;
      // The wait happened because requests in flight had to be assumed to create all their
      // keys. Small tables get room for two more such requests, so that a caller who keeps
      // requests of this size in flight does not wait again on every one of them; for large
      // tables the wait is short next to their kernels and the memory is not.
      const uint64_t slack_n = grown_cap(t, t->base_count + 3 * n) * sizeof(Slot) <= kSlackBytes ? 2 * n : 0;
      const uint64_t slack_u = t->arena_cap * sizeof(float) <= kSlackBytes ? 2 * units : 0;
      if ((double)(t->base_count + n + slack_n) > limit) {
        rc = grow_slots(t, t->base_count + n + slack_n);
        if (rc) return rc;
      }
      if (units && (t->base_top + units + slack_u) * floats_per_unit > t->arena_cap) {
        rc = grow_arena(t, (t->base_top + units + slack_u) * floats_per_unit,
                        t->base_top * floats_per_unit);
        if (rc) return rc;
      }
    }
  }
  const uint64_t q = t->seq++;
  t->log_keys[q % pskv_table::kLog] = n;
  t->log_units[q % pskv_table::kLog] = units;
  t->pend_keys += n;
  t->pend_units += units;
  // Close to a limit every request leaves a record; from a third of the way to the next growth on,
  // every fourth one does (the election of a kernel's last workgroup costs a 1M-key launch about
  // 6 us): the host then knows how full the table is early enough to have the next array allocated
  // by the time it is needed.
  const double limit_now = (double)t->max_load * (double)t->cap;
  const double reach = (double)(t->base_count + t->pend_keys + 2 * n);
  const bool tight_slots = reach > limit_now || (reach > 0.35 * limit_now && q % 4 == 0);
  const bool tight_arena =
      units && (t->base_top + t->pend_units + 2 * units) * floats_per_unit > t->arena_cap;
  // (a base that merely grows old asks for a record every eighth request, not every one)
  const uint64_t age = t->seq - t->base_seq;
  const bool old_base = age >= (uint64_t)pskv_table::kLog / 4 && (age % 8 == 0 || age >= (uint64_t)pskv_table::kLog - 8);
  ++t->stats.requests;
  if (tight_slots || tight_arena || old_base) {
    pub->snap = t->snap;
    pub->seq = q;
    t->record_seq = q;
    ++t->stats.records;
  }
  return PSKV_OK;
}

// ---- request pipeline ------------------------------------------------------------
// One table's share of a request.
struct Request {
  bool push, pull;
  const uint64_t* keys;  // device
  uint64_t n;
  const float* vals;     // device
  uint64_t nvals;
  const int32_t* lens;   // device
  float* out;            // device
  uint64_t out_cap;
  int32_t* out_lens;     // device (VARLEN pull)
  uint64_t out_nvals;    // result
  bool lazy_out;         // VARLEN pull into host memory: `out` is allocated once the size is known
  bool need_total;       // VARLEN pull: the caller wants the response size back (forces a wait)
  char* small_out;       // lazy_out: pinned room the response may go to when it fits
  uint64_t small_out_floats;
  // Large host-resident requests (row modes). pipe_in: `vals` is room in device memory that the
  // row kernel fills itself, piece by piece, from `vals_host` while it works through the pieces
  // that have arrived. pipe_out: the gather kernel is not launched with the request; the caller
  // launches it piece by piece in step with the transfer of the response (gather_deferred says
  // that it is still owed, gather_varlen which kernel it is).
  const float* vals_host;
  bool pipe_in, pipe_out, gather_deferred, gather_varlen;
  // pskv_replay_record: kReplayPrime = the run that brings the tables into the state a repeat of the
  // request finds (the key cache is filled whatever the size of the request and whatever earlier
  // comparisons came to); kReplayCapture = the launches of such a repeat, recorded, not run.
  int replay;
};
constexpr int kReplayPrime = 1, kReplayCapture = 2;

// A request as the kernels see it: the shares of up to kMaxBatch tables that live on one device,
// work in one mode and run on one stream, served by ONE launch per step of the pipeline. The
// single-table entry points run a batch of one; pskv_push_multi / pskv_pull_multi hand over all
// key ranges of a sliced request at once.
struct Item {
  pskv_table* t = nullptr;
  Request r{};
  TableReq d{};
  PublishReq pub;
  ReqTag tag{};
  // var-len workspace of the request
  int32_t* tmp_lens = nullptr;
  uint64_t nparts = 0, tiles_cap = 0;
  // SCALAR: the slots may lag behind the key cache and must be written back if the device finds
  // that this request does not repeat the cached keys
  bool flush_unless_same = false;
};
typedef std::vector<Item> Batch;

// The table whose stream the batch runs on and whose launch statistics it is booked to.
pskv_table* lead_of(Batch& bt) {
  for (Item& it : bt)
    if (it.t->prof) return it.t;
  return bt[0].t;
}

// A launch as pskv_replay_record keeps it: everything hipLaunchKernelGGL needs to make it again.
struct SavedLaunch {
  void (*kernel)(ReqBatch);
  dim3 grid;
  ReqBatch rb;
};
// Where launch_batch leaves a copy of its launches while a request is being recorded (the thread
// that records is the thread that launches).
thread_local std::vector<SavedLaunch>* g_recording = nullptr;

// One launch for the whole batch: blockIdx.y selects the table, `nblk_of` says how many
// workgroups serve each (0: none, the table sits this step out).
template <typename F>
int launch_batch(Batch& bt, int prof_kernel, void (*kernel)(ReqBatch), F nblk_of) {
  ReqBatch rb;
  std::memset(&rb, 0, sizeof(rb));
  uint64_t gx = 0;
  for (size_t i = 0; i < bt.size(); ++i) {
    const uint64_t nb = nblk_of(bt[i]);
    if (nb > 0x7fffffffull) return set_error(PSKV_EINVAL, "request too large");
    rb.t[i] = bt[i].d;
    rb.t[i].nblk = (uint32_t)nb;
    gx = std::max(gx, nb);
  }
  if (!gx) return PSKV_OK;
  launch(lead_of(bt), prof_kernel, kernel, dim3((unsigned)gx, (unsigned)bt.size()), dim3(kBlock), rb);
  PSKV_HIP(hipGetLastError());
  if (g_recording) g_recording->push_back(SavedLaunch{kernel, dim3((unsigned)gx, (unsigned)bt.size()), rb});
  return PSKV_OK;
}

// The device state of every table of the batch with one launch and one wait.
int read_state_batch(Batch& bt) {
  StateBatch sb;
  std::memset(&sb, 0, sizeof(sb));
  for (size_t i = 0; i < bt.size(); ++i) {
    sb.st[i] = bt[i].t->st;
    sb.out[i] = bt[i].t->st_host;
  }
  k_read_state<<<dim3((unsigned)bt.size()), dim3(64), 0, bt[0].t->stream>>>(sb);
  PSKV_HIP(hipGetLastError());
  PSKV_HIP(hipStreamSynchronize(bt[0].t->stream));
  for (Item& it : bt) adopt_state(it.t);
  return PSKV_OK;
}

// What the device has reported about the comparisons of earlier requests with the cached keys
// (a pinned word, read whenever the host gets here, never waited for): comparisons that keep
// finding other keys switch the comparison off for 2, 4, ... 64 requests of that kind.
void note_outcomes(pskv_table* t) {
  const unsigned long long seen = *static_cast<volatile unsigned long long*>(t->outcome);
  if (seen == t->sc_seen) return;
  t->sc_seen = seen;
  const unsigned long long e = seen >> 1;
  if (e + pskv_table::kScKinds <= t->epoch) return;  // the note of its kind has been overwritten
  pskv_table::ScTrack& tr = t->sc_track[t->sc_kind[e % pskv_table::kScKinds] & 1];
  if (seen & 1ull) {
    tr.fail = 0;
    tr.hit = true;
  } else {
    tr.fail = std::min(tr.fail + 1u, 6u);
    tr.skip = 1u << tr.fail;
    tr.hit = false;
  }
}

// Numbers a request that takes part in the key cache and says whether the key cache has the
// right shape for it. Row modes (`back_off`): a request of the right shape is still not compared
// while comparisons of its kind (pushes, pulls) are in a spell of finding other keys, as the
// requests of an embedding table do that names other rows in every batch; the request then goes
// the general way, which leaves its keys behind as the new cache all the same.
ReqTag next_tag(pskv_table* t, const Request& r, bool back_off = false) {
  ReqTag tag;
  tag.epoch = ++t->epoch;
  tag.replay = r.replay == kReplayCapture ? 1u : 0u;
  bool compare = t->cache_valid && t->cache_n == r.n;
  if (back_off && compare && !r.replay) {
    note_outcomes(t);
    const int kind = r.push ? 0 : 1;
    pskv_table::ScTrack& tr = t->sc_track[kind];
    if (tr.skip) {
      --tr.skip;
      compare = false;
    } else {
      t->sc_kind[tag.epoch % pskv_table::kScKinds] = (unsigned char)kind;
    }
  }
  tag.try_cache = compare ? 1u : 0u;
  return tag;
}

// SCALAR requests of at least this many keys may use the key cache (below that a request is a
// single short launch either way, and the cache would add two). The environment variable
// PSKV_SCALAR_CACHE_MIN_KEYS, read when a table is created, overrides it (0 switches the cache off).
constexpr uint64_t kScalarCacheMinKeys = 1u << 17;

// How a SCALAR request of one table relates to the table's key cache.
enum ScalarCacheUse {
  kScPlain,   // neither uses nor fills it
  kScRecord,  // served through the slots; leaves its keys, values and slot numbers as the new cache
  kScTry,     // compared with the cached keys on the device: served from the cache if they match,
              // like kScRecord otherwise
};

// Decides it from what the host knows without waiting for the device: a request whose size
// repeats the previous one is worth recording, a request of the cached size is worth comparing,
// and comparisons that keep finding other keys (reported by the device through a pinned word,
// read whenever the host gets here) switch the comparison off for a growing number of requests
// of that kind.
bool scalar_cache_eligible(const pskv_table* t, const Request& r) {
  return t->sc_min_keys && r.n >= t->sc_min_keys && t->cap < (1ull << 32);
}

ScalarCacheUse scalar_cache_use(pskv_table* t, const Request& r) {
  note_outcomes(t);
  const int kind = r.push ? 0 : 1;
  // a worker that pushes gradients and pulls the weights of the same keys right away shows as a
  // pull behind a push of its own size, whatever that size is from one step to the next
  if (kind == 1 && t->sc_last_kind == 0)
    t->sc_pairs = r.n == t->sc_last_n ? std::min(t->sc_pairs + 1u, 2u) : 0u;
  ScalarCacheUse use = kScPlain;
  if (scalar_cache_eligible(t, r)) {
    pskv_table::ScTrack& tr = t->sc_track[kind];
    const bool compare = tr.skip == 0;
    if (!compare) --tr.skip;
    const bool size_repeats = r.n == t->sc_last_n;
    if (compare && t->cache_valid && t->cache_n == r.n) {
      use = kScTry;
    } else if (kind == 0) {
      // a push is worth recording when its size repeats (the same keys may be coming again) or
      // when pulls have been following the pushes and are not in a spell of failed comparisons
      const bool pulls_follow = t->sc_pairs >= 2 && t->sc_track[1].skip == 0;
      if ((compare && size_repeats) || pulls_follow) use = kScRecord;
    } else if (compare && size_repeats && t->sc_last_kind == 1) {
      use = kScRecord;  // a pull behind a pull of the same size
    }
  }
  t->sc_last_n = r.n;
  t->sc_last_kind = kind;
  return use;
}

int run_scalar(Batch& bt, bool push, bool pull) {
  uint64_t n_largest = 0;
  bool any_cache = false;
  std::vector<ScalarCacheUse> use(bt.size(), kScPlain);
  for (size_t i = 0; i < bt.size(); ++i) {
    Item& it = bt[i];
    pskv_table* t = it.t;
    Request& r = it.r;
    r.out_nvals = pull ? r.n : 0;
    it.d = TableReq{};
    if (r.n == 0) continue;
    // (a growth writes the cache back and drops it; a recorded repeat creates no key)
    int rc = r.replay == kReplayCapture ? PSKV_OK : reserve(t, r.n, 0, 0, &it.pub);
    if (rc) return rc;
    const int kind_before = t->sc_last_kind;
    if (r.replay) {
      // a request that is being recorded fills the key cache, or is compared with it, whatever its size
      if (t->cap >= (1ull << 32))
        return set_error(PSKV_EINVAL, "a table of 2^32 slots keeps no key cache: its requests cannot be recorded");
      const bool fits = t->cache_valid && t->cache_n == r.n;
      if (r.replay == kReplayCapture && !fits)
        return set_error(PSKV_ESTALE, "the key cache does not hold the request that is being recorded");
      use[i] = fits ? kScTry : kScRecord;
      t->sc_last_n = r.n;
      t->sc_last_kind = r.push ? 0 : 1;
    } else {
      use[i] = scalar_cache_use(t, r);
    }
    if (use[i] != kScTry) {
      // the request goes through the slots, so they must be up to date; a push then makes the
      // cached values stale, a recording replaces them
      rc = flush_scalar_cache(t);
      if (rc) return rc;
      if (push || use[i] == kScRecord) t->cache_valid = false;
    }
    TableReq& d = it.d;
    if (use[i] == kScRecord) {
      // Room for this request in the cache (it has been written back above; kScTry needs nothing:
      // the buffers have the cached request's size). Only a request that is going to be recorded
      // pays for it: a one-off pull of 16M keys would otherwise allocate 256 MB it never uses, and
      // wait for the stream to do so.
      rc = grow(t, &t->cache_keys, r.n * sizeof(uint64_t));
      if (rc) return rc;
      rc = grow(t, &t->sc_vals, r.n * sizeof(float));
      if (rc) return rc;
      rc = grow(t, &t->sc_slots, r.n * sizeof(uint32_t));
      if (rc) return rc;
    }
    if (use[i] != kScPlain) {
      it.tag = next_tag(t, r);
      t->sc_kind[it.tag.epoch % pskv_table::kScKinds] = r.push ? 0 : 1;
      d.tag = it.tag;
      d.cache_keys = static_cast<uint64_t*>(t->cache_keys.ptr);
      d.arena = static_cast<float*>(t->sc_vals.ptr);
      d.tile_key = static_cast<uint32_t*>(t->sc_slots.ptr);
      d.outcome = t->outcome;
      // A pull right behind a push, with the slots up to date (the push went through them and
      // recorded itself): the pull kernel compares key by key and needs no launch in front of it.
      // (not in a recording: keys that differ would go through the slots there)
      const bool per_key = use[i] == kScTry && !push && !t->sc_dirty && kind_before == 0 && r.replay != kReplayCapture;
      d.cache_mode = per_key ? kCachePerKey : kCacheOn;
      any_cache = true;
      // (a recorded repeat is served from the cache or not at all: nothing to write back first)
      it.flush_unless_same = !per_key && it.tag.try_cache && t->sc_dirty && r.replay != kReplayCapture;
    }
    d.slots = t->slots;
    d.mask = t->cap - 1;
    d.st = t->st;
    d.keys = r.keys;
    d.vals = r.vals;
    d.out = r.out;
    d.n = r.n;
    d.snap = it.pub.snap;  // the request's kernel leaves the counter record itself
    d.snap_seq = it.pub.seq;
    n_largest = std::max(n_largest, r.n);
  }
  if (!n_largest) return PSKV_OK;
  int rc;
  if (any_cache) {
    rc = launch_batch(bt, PSKV_KERNEL_SAME_KEYS, k_same_keys, [](const Item& it) {
      return (it.d.cache_mode == kCacheOn && it.tag.try_cache)
                 ? (it.r.n + kBlock * kSameKeysItems - 1) / (kBlock * kSameKeysItems) : 0ull;
    });
    if (rc) return rc;
    // slots that lag behind the cache are written back once the device knows that the request
    // does NOT repeat the cached keys (cache_mode reads as kFlushUnlessSame in that kernel)
    static_assert(kFlushUnlessSame == kCacheOn, "one descriptor serves both kernels");
    rc = launch_batch(bt, -1, k_scalar_flush, [](const Item& it) {
      return it.flush_unless_same ? (uint64_t)grid_for(it.r.n, kBlock, kFlushGrid) : 0ull;
    });
    if (rc) return rc;
  }
  // The kernel strides over a table's keys, so a grid capped at kMaxGrid serves any request. A
  // request that is expected to repeat the cached keys gets a quarter of the workgroups: served
  // from the cache it moves four keys per lane (should it go through the slots after all, every
  // lane takes four turns).
  auto nblk = [&](const Item& it) -> uint64_t {
    if (!it.d.n) return 0;
    const bool four = (it.d.cache_mode == kCacheOn && it.tag.try_cache) || it.d.cache_mode == kCachePerKey;
    return grid_for(it.d.n, four ? kBlock * 4 : kBlock, kMaxGrid);
  };
  if (push && pull) {
    rc = any_cache ? launch_batch(bt, PSKV_KERNEL_PUSH_SCALAR, k_scalar<true, true, true>, nblk)
                   : launch_batch(bt, PSKV_KERNEL_PUSH_SCALAR, k_scalar<true, true, false>, nblk);
  } else if (push) {
    rc = any_cache ? launch_batch(bt, PSKV_KERNEL_PUSH_SCALAR, k_scalar<true, false, true>, nblk)
                   : launch_batch(bt, PSKV_KERNEL_PUSH_SCALAR, k_scalar<true, false, false>, nblk);
  } else {
    const int kind = bt[0].d.cache_mode == kCachePerKey ? PSKV_KERNEL_PULL_PER_KEY : PSKV_KERNEL_PULL_SCALAR;
    rc = any_cache ? launch_batch(bt, kind, k_scalar<false, true, true>, nblk)
                   : launch_batch(bt, PSKV_KERNEL_PULL_SCALAR, k_scalar<false, true, false>, nblk);
  }
  if (rc) return rc;
  for (size_t i = 0; i < bt.size(); ++i) {
    if (use[i] == kScPlain || !bt[i].r.n) continue;
    pskv_table* t = bt[i].t;
    t->cache_valid = true;  // whichever way the device decides, the cache now stands for this request
    t->cache_n = bt[i].r.n;
    if (push && use[i] == kScTry) t->sc_dirty = true;  // served from the cache: the slots lag behind
  }
  return PSKV_OK;
}

// Requests at least this large (4 MiB) are streamed with non-temporal accesses: between two
// requests of a busy server they do not survive in the caches anyway.
constexpr uint64_t kStreamFloats = 1u << 20;

// The row kernel over `floats` request-side floats of the batch's only table, starting at float
// `first` (a multiple of the tile size): one piece of a request that is served as it arrives.
template <bool VARLEN>
int launch_rows_piece(Batch& bt, int op, uint64_t first, uint64_t floats) {
  const uint64_t tile = VARLEN ? kRowsVarPerBlock : kTileFixed;
  Item& it = bt[0];
  const bool stream = it.d.total >= kStreamFloats;
  it.d.tile_base = (uint32_t)(first / tile);
  auto nblk = [&](const Item&) { return (floats + tile - 1) / tile; };
  int rc;
  if (op == kOpAcc) {
    rc = stream ? launch_batch(bt, PSKV_KERNEL_ROWS_ACC, k_rows<kOpAcc, VARLEN, true>, nblk)
                : launch_batch(bt, PSKV_KERNEL_ROWS_ACC, k_rows<kOpAcc, VARLEN, false>, nblk);
  } else {
    rc = stream ? launch_batch(bt, PSKV_KERNEL_ROWS_GATHER, k_rows<kOpGather, VARLEN, true>, nblk)
                : launch_batch(bt, PSKV_KERNEL_ROWS_GATHER, k_rows<kOpGather, VARLEN, false>, nblk);
  }
  it.d.tile_base = 0;
  return rc;
}

// The row kernel over every table of the batch whose TableReq::total is not zero.
template <bool VARLEN>
int launch_rows(Batch& bt, int op) {
  const uint64_t tile = VARLEN ? kRowsVarPerBlock : kTileFixed;  // request-side floats per workgroup
  uint64_t floats = 0;
  for (const Item& it : bt) floats += it.d.total;
  if (!floats) return PSKV_OK;
  if (bt.size() == 1 && op == kOpAcc && bt[0].r.pipe_in) {
    // the values are still in the caller's memory: every piece is accumulated as soon as it is here
    Item& it = bt[0];
    Stager* sg = Stager::get(it.t->device);
    if (!sg) return set_error(PSKV_ENOMEM, "no pinned memory to stage the request through");
    return sg->to_device(const_cast<float*>(it.r.vals), it.r.vals_host, it.d.total * sizeof(float),
                         it.t->stream, [&](size_t off, size_t len) {
                           return launch_rows_piece<VARLEN>(bt, kOpAcc, off / sizeof(float), len / sizeof(float));
                         });
  }
  if (bt.size() == 1 && op == kOpGather && bt[0].r.pipe_out) {
    bt[0].r.gather_deferred = true;  // launched piece by piece in step with the transfer to the host
    bt[0].r.gather_varlen = VARLEN;
    return PSKV_OK;
  }
  auto nblk = [&](const Item& it) { return (it.d.total + tile - 1) / tile; };
  const bool stream = floats >= kStreamFloats;
  if (op == kOpAcc) {
    if (stream) return launch_batch(bt, PSKV_KERNEL_ROWS_ACC, k_rows<kOpAcc, VARLEN, true>, nblk);
    return launch_batch(bt, PSKV_KERNEL_ROWS_ACC, k_rows<kOpAcc, VARLEN, false>, nblk);
  }
  if (stream) return launch_batch(bt, PSKV_KERNEL_ROWS_GATHER, k_rows<kOpGather, VARLEN, true>, nblk);
  return launch_batch(bt, PSKV_KERNEL_ROWS_GATHER, k_rows<kOpGather, VARLEN, false>, nblk);
}

// Starts a row-mode request on every table with keys: numbers it and, where the key cache has
// the right shape, lets the device compare the request with the cached one. Call after every
// buffer the cache lives in has been grown for this request.
int begin_row_request(Batch& bt) {
  for (Item& it : bt) {
    if (!it.r.n) continue;
    it.tag = next_tag(it.t, it.r, true);
    if (it.r.replay == kReplayCapture && !it.tag.try_cache)
      return set_error(PSKV_ESTALE, "the key cache does not hold the request that is being recorded%s",
                       it.t->mode == PSKV_MODE_VARLEN ? " (a PSKV_MODE_VARLEN pull leaves no key cache behind: record "
                                                        "it together with the push of its keys, or right behind one)"
                                                      : "");
    it.d.tag = it.tag;
    it.d.outcome = it.t->outcome;
  }
  return launch_batch(bt, PSKV_KERNEL_SAME_KEYS, k_same_keys, [](const Item& it) {
    return (it.r.n && it.tag.try_cache) ? (it.r.n + kBlock * kSameKeysItems - 1) / (kBlock * kSameKeysItems)
                                        : 0ull;
  });
}

int run_fixed(Batch& bt, bool push, bool pull) {
  uint64_t n_largest = 0;
  for (Item& it : bt) {
    pskv_table* t = it.t;
    Request& r = it.r;
    const uint64_t k = t->row_len;
    r.out_nvals = pull ? r.n * k : 0;
    it.d = TableReq{};
    if (r.n == 0) continue;
    int rc = r.replay == kReplayCapture ? PSKV_OK : reserve(t, r.n, r.n, k, &it.pub);
    if (rc) return rc;
    rc = grow(t, &t->ws, Carver::need(r.n, sizeof(uint64_t)));
    if (rc) return rc;
    rc = grow(t, &t->cache_keys, r.n * sizeof(uint64_t));
    if (rc) return rc;
    Carver c(t->ws.ptr);
    TableReq& d = it.d;
    d.slots = t->slots;
    d.mask = t->cap - 1;
    d.st = t->st;
    d.keys = r.keys;
    d.n = r.n;
    d.arena = t->arena;
    d.ref = c.take<uint64_t>(r.n);
    d.cache_keys = static_cast<uint64_t*>(t->cache_keys.ptr);
    d.snap = it.pub.snap;
    d.snap_seq = it.pub.seq;
    d.k = k;
    n_largest = std::max(n_largest, r.n);
  }
  if (!n_largest) return PSKV_OK;
  int rc = begin_row_request(bt);
  if (rc) return rc;
  if (bt[0].r.replay == kReplayCapture) {
    // a recorded repeat uses the references that are there: no lookup
  } else if (n_largest >= kLookupLargeKeys) {
    rc = launch_batch(bt, PSKV_KERNEL_LOOKUP, k_lookup_fixed<kLookupItemsLarge>, [](const Item& it) {
      return it.r.n ? (uint64_t)grid_for(it.r.n, kBlock * kLookupItemsLarge, kMaxGrid) : 0ull;
    });
  } else {
    rc = launch_batch(bt, PSKV_KERNEL_LOOKUP, k_lookup_fixed<1>, [](const Item& it) {
      return it.r.n ? (uint64_t)grid_for(it.r.n, kBlock, kMaxGrid) : 0ull;
    });
  }
  if (rc) return rc;
  for (Item& it : bt) {
    if (!it.r.n) continue;
    // push and pull both create absent keys, so either leaves references for all n keys behind
    it.t->cache_valid = true;
    it.t->cache_n = it.r.n;
    it.t->cache_nvals = it.r.n * it.d.k;
  }
  if (push) {
    for (Item& it : bt) {
      if (!it.r.n) continue;
      it.d.req = const_cast<float*>(it.r.vals);
      it.d.total = it.r.n * it.d.k;
      it.d.force_scalar = ((it.d.k & 3) || (reinterpret_cast<uintptr_t>(it.r.vals) & 15)) ? 1u : 0u;
      it.d.ignore_new = 0;
    }
    rc = launch_rows<false>(bt, kOpAcc);
    if (rc) return rc;
  }
  if (pull) {
    for (Item& it : bt) {
      if (!it.r.n) continue;
      it.d.req = it.r.out;
      it.d.total = it.r.n * it.d.k;
      it.d.force_scalar = ((it.d.k & 3) || (reinterpret_cast<uintptr_t>(it.r.out) & 15)) ? 1u : 0u;
      it.d.ignore_new = push ? 1u : 0u;
    }
    rc = launch_rows<false>(bt, kOpGather);
    if (rc) return rc;
  }
  return PSKV_OK;
}

// Room in the two tile tables for `floats` request-side floats.
int grow_tile_tables(pskv_table* t, uint64_t floats, uint64_t* ntiles_cap) {
  *ntiles_cap = (floats + kTileVar - 1) / kTileVar;
  int rc = grow(t, &t->tiles, (*ntiles_cap + 1) * sizeof(uint32_t));
  if (rc) return rc;
  return grow(t, &t->tiles_aff, (*ntiles_cap + 1) * sizeof(TileNote));
}

// The kernels of a var-len request that work key by key: one workgroup per kBlock*items keys,
// `items` per thread, the same split in every kernel of the request and for every table of the
// batch (the scan's per-workgroup totals are indexed by it).
int launch_keys(Batch& bt, int prof_kernel, int items, void (*k1)(ReqBatch), void (*k4)(ReqBatch)) {
  return launch_batch(bt, prof_kernel, items == kScanItemsLarge ? k4 : k1,
                      [](const Item& it) { return it.r.n ? it.nparts : 0ull; });
}

// Pass 2 of a pull's scan for every table with a response: the request-side offsets of the
// response and the tile table for Item::d.total floats of room (the row kernel fills the other
// table).
int make_tile_tables(Batch& bt, int items) {
  for (Item& it : bt) {
    if (!it.d.total) continue;
    uint64_t ntiles_cap = 0;
    int rc = grow_tile_tables(it.t, it.d.total, &ntiles_cap);
    if (rc) return rc;
    it.d.tile_key = static_cast<uint32_t*>(it.t->tiles.ptr);
    it.d.tile_aff = static_cast<TileNote*>(it.t->tiles_aff.ptr);
    it.d.ntiles = ntiles_cap;
  }
  if (bt[0].r.replay == kReplayCapture) return PSKV_OK;  // (a recorded repeat: the tables that are there)
  return launch_batch(bt, -1, items == kScanItemsLarge ? k_var_offsets<kScanItemsLarge> : k_var_offsets<1>,
                      [](const Item& it) { return (it.r.n && it.d.total) ? it.nparts : 0ull; });
}

// Launches per var-len request: a push takes three (compare + scan pass 1; scan pass 2 +
// find-or-create + counter record; rows), a pull four (compare; stored lengths + scan pass 1;
// scan pass 2 + tile table; rows), whatever the number of tables.
int run_varlen(Batch& bt, bool push, bool pull) {
  uint64_t n_largest = 0;
  for (Item& it : bt) {
    it.r.out_nvals = 0;
    it.d = TableReq{};
    if (it.r.n > 0xfffffffeull) return set_error(PSKV_EINVAL, "too many keys in one request");
    n_largest = std::max(n_largest, it.r.n);
  }
  if (!n_largest) return PSKV_OK;
  // (keys per thread of the key-by-key kernels: by the keys of the whole launch, not of its largest table)
  uint64_t n_launch = 0;
  for (const Item& it : bt) n_launch += it.r.n;
  const int items = scan_items(n_launch);
  const bool async_pull = pull && !push && !bt[0].r.need_total;
  for (Item& it : bt) {
    pskv_table* t = it.t;
    Request& r = it.r;
    if (!r.n) continue;
    it.nparts = scan_num_parts(r.n, items);
    const size_t need = Carver::need(r.n, 8) + Carver::need(r.n + 1, 8) + Carver::need(it.nparts, 8) +
                        Carver::need(r.n, 4);
    // Every buffer the key cache lives in is grown BEFORE the request is compared with the
    // cached one: a reallocation loses the cached contents and must rule the fast path out.
    int rc = grow(t, &t->ws, need);
    if (rc) return rc;
    rc = grow(t, &t->cache_keys, r.n * sizeof(uint64_t));
    if (rc) return rc;
    rc = grow(t, &t->cache_lens, r.n * sizeof(int32_t));
    if (rc) return rc;
    const uint64_t tiles_for = push ? r.nvals : (async_pull ? r.out_cap : 0);
    rc = grow_tile_tables(t, tiles_for, &it.tiles_cap);
    if (rc) return rc;
    Carver c(t->ws.ptr);
    TableReq& d = it.d;
    d.ref = c.take<uint64_t>(r.n);
    d.off = c.take<uint64_t>(r.n + 1);
    d.part = c.take<unsigned long long>(it.nparts);
    it.tmp_lens = c.take<int32_t>(r.n);
    d.cache_keys = static_cast<uint64_t*>(t->cache_keys.ptr);
    d.cache_lens = static_cast<int32_t*>(t->cache_lens.ptr);
    d.keys = r.keys;
    d.n = r.n;
    d.st = t->st;
  }

  if (push) {
    for (Item& it : bt) {
      pskv_table* t = it.t;
      Request& r = it.r;
      if (!r.n) continue;
      // every key may round its row up to a 16-byte unit, every workgroup may pad its rows' start
      int rc = r.replay == kReplayCapture
                   ? PSKV_OK
                   : reserve(t, r.n, r.nvals / 4 + r.n + kArenaPadUnits * it.nparts, 4, &it.pub);
      if (rc) return rc;
      if (t->cache_nvals != r.nvals) t->cache_valid = false;  // same lens would mean the same total
      it.tag = next_tag(t, r, true);
      if (r.replay == kReplayCapture && !it.tag.try_cache)
        return set_error(PSKV_ESTALE, "the key cache does not hold the request that is being recorded");
      TableReq& d = it.d;
      d.outcome = t->outcome;
      d.slots = t->slots;
      d.mask = t->cap - 1;
      d.arena = t->arena;
      d.lens = r.lens;
      d.nvals = r.nvals;
      d.tag = it.tag;
      d.snap = it.pub.snap;
      d.snap_seq = it.pub.seq;
      // pass 2 also fills the tile table of the request side (tile sizes are those of nvals; a
      // request whose lens do not add up to nvals is refused before it gets there)
      d.tile_key = r.nvals ? static_cast<uint32_t*>(t->tiles.ptr) : nullptr;
      d.tile_aff = static_cast<TileNote*>(t->tiles_aff.ptr);
      d.ntiles = it.tiles_cap;
    }
    int rc = launch_keys(bt, -1, items, k_var_push_begin<1>, k_var_push_begin<kScanItemsLarge>);
    if (rc) return rc;
    // (a recorded repeat uses the offsets, tile table and references that are there)
    if (bt[0].r.replay != kReplayCapture)
      rc = launch_keys(bt, PSKV_KERNEL_LOOKUP, items, k_var_push_lookup<1>, k_var_push_lookup<kScanItemsLarge>);
    if (rc) return rc;
    for (Item& it : bt) {
      if (!it.r.n) continue;
      it.t->cache_valid = true;  // whichever way the device decided, the cache now is this request
      it.t->cache_n = it.r.n;
      it.t->cache_nvals = it.r.nvals;
      it.d.req = const_cast<float*>(it.r.vals);
      it.d.total = it.r.nvals;
      it.d.force_scalar = (reinterpret_cast<uintptr_t>(it.r.vals) & 15) ? 1u : 0u;
      it.d.ignore_new = 0;
      it.d.total_on_device = 0;
    }
    rc = launch_rows<true>(bt, kOpAcc);
    if (rc) return rc;
  }
  if (pull) {
    int rc;
    if (push) {
      // a refused push must not be followed by its pull half
      rc = read_state_batch(bt);
      if (rc) return rc;
      for (Item& it : bt) {
        rc = report_device_errors(it.t);
        if (rc) return rc;
      }
    }
    for (Item& it : bt) {
      if (!it.r.n) continue;
      it.d.slots = it.t->slots;
      it.d.mask = it.t->cap - 1;
      it.d.arena = it.t->arena;
      it.d.out_lens = it.r.out_lens ? it.r.out_lens : it.tmp_lens;
      it.d.total = 0;
      it.d.snap = nullptr;
    }
    // A pull with the keys of the cached push finds every key present with the cached length
    // and reuses its references; any other pull recomputes them and so ends the cache.
    rc = begin_row_request(bt);
    if (rc) return rc;
    for (Item& it : bt)
      if (it.r.n && !it.tag.try_cache) it.t->cache_valid = false;
    rc = launch_keys(bt, PSKV_KERNEL_LOOKUP, items, k_var_pull_lookup<1>, k_var_pull_lookup<kScanItemsLarge>);
    if (rc) return rc;
    if (async_pull) {
      // No host round trip: the grid covers the caller's buffer, the kernels take the real
      // size from the scan, and a response that does not fit is reported by the next sync.
      for (Item& it : bt) {
        if (!it.r.n || !it.r.out_cap) continue;
        if (!it.r.out) return set_error(PSKV_EINVAL, "null out");
        it.d.req = it.r.out;
        it.d.total = it.r.out_cap;
        it.d.total_on_device = 1;
        it.d.force_scalar = (reinterpret_cast<uintptr_t>(it.r.out) & 15) ? 1u : 0u;
        it.d.ignore_new = 1;
      }
      rc = make_tile_tables(bt, items);
      if (rc) return rc;
      return launch_rows<true>(bt, kOpGather);
    }
    rc = read_state_batch(bt);  // the response sizes are data dependent
    if (rc) return rc;
    int fit = PSKV_OK;
    for (Item& it : bt) {
      pskv_table* t = it.t;
      Request& r = it.r;
      if (!r.n) continue;
      if (t->st_host->same_epoch != it.tag.epoch) t->cache_valid = false;  // the pull recomputed the workspace
      const uint64_t total = t->st_host->scan_total;
      r.out_nvals = total;
      if (total > r.out_cap && !fit)
        fit = set_error(PSKV_ESIZE_MISMATCH, "response needs %llu floats, buffer holds %llu",
                        (unsigned long long)total, (unsigned long long)r.out_cap);
    }
    if (fit) return fit;
    for (Item& it : bt) {
      pskv_table* t = it.t;
      Request& r = it.r;
      const uint64_t total = r.n ? r.out_nvals : 0;
      if (!total) continue;
      if (r.lazy_out) {
        if (r.small_out && total <= r.small_out_floats) {
          r.out = reinterpret_cast<float*>(r.small_out);
        } else {
          rc = grow(t, &t->stage_out, total * sizeof(float));
          if (rc) return rc;
          r.out = static_cast<float*>(t->stage_out.ptr);
        }
      }
      if (!r.out) return set_error(PSKV_EINVAL, "null out");
      it.d.req = r.out;
      it.d.total = total;
      it.d.total_on_device = 0;
      it.d.force_scalar = (reinterpret_cast<uintptr_t>(r.out) & 15) ? 1u : 0u;
      it.d.ignore_new = 1;
    }
    rc = make_tile_tables(bt, items);
    if (rc) return rc;
    rc = launch_rows<true>(bt, kOpGather);
    if (rc) return rc;
  }
  return PSKV_OK;
}

int run_batch(Batch& bt, bool push, bool pull) {
  int rc;
  const bool capturing = bt[0].t->capturing;
  if (!capturing)
    for (Item& it : bt) ++it.t->gen;
  switch (bt[0].t->mode) {
    case PSKV_MODE_SCALAR: rc = run_scalar(bt, push, pull); break;
    case PSKV_MODE_FIXED: rc = run_fixed(bt, push, pull); break;
    default: rc = run_varlen(bt, push, pull); break;
  }
  // the GPU is busy with the request now: the moment to allocate ahead of a coming growth
  if (!rc && !capturing)
    for (Item& it : bt) prepare_growth(it.t);
  return rc;
}

// Host-side checks that mirror the CHECKs of the reference and the frozen rules of
// the row modes; nothing is enqueued when they fail.
int validate(pskv_table* t, bool push, bool pull, uint64_t n, uint64_t nvals, const int32_t* lens,
             uint64_t nlens, int memkind) {
  switch (t->mode) {
    case PSKV_MODE_SCALAR:
      // kv_app.h:447 CHECK_EQ(n, req_data.vals.size()); with pull set the reference
      // indexes vals[i] unchecked, which this library refuses when the sizes differ
      if (push && n != nvals)
        return set_error(PSKV_ESIZE_MISMATCH, "%llu keys but %llu values", (unsigned long long)n,
                         (unsigned long long)nvals);
      return PSKV_OK;
    case PSKV_MODE_FIXED:
      if (push) {
        if (n == 0) {
          if (nvals) return set_error(PSKV_ESIZE_MISMATCH, "values without keys");
        } else {
          const uint64_t k = nvals / n;  // kv_app.h:548-549
          if (k * n != nvals || k == 0)
            return set_error(PSKV_ESIZE_MISMATCH, "%llu values do not divide over %llu keys",
                             (unsigned long long)nvals, (unsigned long long)n);
          if (t->row_len == 0) t->row_len = k;
          if (k != t->row_len)
            return set_error(PSKV_ESIZE_MISMATCH, "row length %llu, table holds rows of %llu",
                             (unsigned long long)k, (unsigned long long)t->row_len);
        }
      }
      if (n && t->row_len == 0) return set_error(PSKV_EINVAL, "pull before the row length is known");
      return PSKV_OK;
    default:
      if (push) {
        if (nlens != n)  // kv_app.h:489,551
          return set_error(PSKV_ESIZE_MISMATCH, "%llu keys but %llu lens", (unsigned long long)n,
                           (unsigned long long)nlens);
        if (n && !lens) return set_error(PSKV_EINVAL, "lens missing");
        if (n == 0 && nvals) return set_error(PSKV_ESIZE_MISMATCH, "values without keys");
        if (memkind == PSKV_MEM_HOST) {
          uint64_t total = 0;
          for (uint64_t i = 0; i < n; ++i) {
            if (lens[i] < 0 || (uint32_t)lens[i] > PSKV_MAX_VARLEN_ROW)
              return set_error(PSKV_EINVAL, "lens[%llu] = %d out of range", (unsigned long long)i,
                               lens[i]);
            total += (uint64_t)lens[i];
          }
          if (total != nvals)
            return set_error(PSKV_ESIZE_MISMATCH, "lens add up to %llu, %llu values given",
                             (unsigned long long)total, (unsigned long long)nvals);
        }
      }
      return PSKV_OK;
  }
}

int request(pskv_table* t, bool push, bool pull, const uint64_t* keys, size_t n, const float* vals,
            size_t nvals, const int32_t* lens, size_t nlens, float* out, size_t out_cap,
            int32_t* out_lens, size_t* out_nvals, int memkind) {
  clear_error();
  if (!t) return set_error(PSKV_EINVAL, "null table");
  if (memkind != PSKV_MEM_HOST && memkind != PSKV_MEM_DEVICE)
    return set_error(PSKV_EINVAL, "bad memkind %d", memkind);
  if (n && !keys) return set_error(PSKV_EINVAL, "null keys");
  if (push && nvals && !vals) return set_error(PSKV_EINVAL, "null vals");
  if (out_nvals) *out_nvals = 0;
  DeviceGuard guard(t->device);
  if (!guard.ok()) return set_error(PSKV_EHIP, "cannot select device %d", t->device);
  int rc = validate(t, push, pull, n, nvals, lens, nlens, memkind);
  if (rc) return rc;
  const bool host = memkind == PSKV_MEM_HOST;
  const bool varlen = t->mode == PSKV_MODE_VARLEN;
  bool small = false;        // host-resident request served from the pinned buffers
  int small_part = -1;       // the part of small_in it lies in when it does not take all of it
  size_t small_out_at = 0;   // bytes of small_out already given away

  // SCALAR and FIXED know the response size up front. A response that does not fit is
  // still computed (into scratch) so that the store ends up as the reference's would:
  // a pull creates absent keys (kv_app.h:457).
  uint64_t fixed_out = 0;
  if (pull && !varlen) fixed_out = t->mode == PSKV_MODE_SCALAR ? n : n * t->row_len;
  const bool too_small = pull && !varlen && fixed_out > out_cap;
  if (pull && !varlen && fixed_out && !too_small && !out) return set_error(PSKV_EINVAL, "null out");

  Request r{};
  r.push = push;
  r.pull = pull;
  r.n = n;
  r.nvals = push ? nvals : 0;
  r.out_cap = out_cap;
  r.need_total = host || out_nvals != nullptr || push;
  if (!host) {
    r.keys = keys;
    r.vals = vals;
    r.lens = lens;
    r.out = out;
    r.out_lens = out_lens;
  } else {
    const bool want_lens = push && varlen;
    const bool want_out_lens = pull && varlen;
    const size_t in_need =
        Carver::need(n, 8) + Carver::need(r.nvals, 4) + Carver::need(want_lens ? n : 0, 4);
    const size_t out_lens_need = Carver::need(want_out_lens ? n : 0, 4);
    small = in_need <= kSmallBytes && out_lens_need <= kSmallBytes;
    char* base = t->small_in;
    // a push that returns at once takes one part of the pinned buffer, the others all of it
    const bool early = small && t->mode == PSKV_MODE_SCALAR && !pull && t->small_done[0] != nullptr;
    small_part = (early && in_need <= kSmallBytes / kSmallParts) ? t->small_next : -1;
    if (small_part >= 0) base += (size_t)small_part * (kSmallBytes / kSmallParts);
    if (!small) {
      rc = grow(t, &t->stage, in_need + out_lens_need);
      if (rc) return rc;
      base = static_cast<char*>(t->stage.ptr);
    }
    Carver c(base);
    uint64_t* dkeys = c.take<uint64_t>(n);
    float* dvals = c.take<float>(r.nvals);
    int32_t* dlens = c.take<int32_t>(want_lens ? n : 0);
    int32_t* dout_lens = nullptr;
    if (small) {
      // earlier requests are done with what this one overwrites: they ended with a wait, or left an event
      if (small_part >= 0) {
        if (t->small_pending[small_part]) {
          PSKV_HIP(hipEventSynchronize(t->small_done[small_part]));
          t->small_pending[small_part] = false;
        }
      } else if (t->small_newest >= 0) {
        PSKV_HIP(hipEventSynchronize(t->small_done[t->small_newest]));  // (one stream: the others came before)
        for (int q = 0; q < kSmallParts; ++q) t->small_pending[q] = false;
        t->small_newest = -1;
      }
      if (n) std::memcpy(dkeys, keys, n * 8);
      if (r.nvals) std::memcpy(dvals, vals, r.nvals * 4);
      if (want_lens && n) std::memcpy(dlens, lens, n * 4);
      small_out_at = out_lens_need;
      if (want_out_lens) dout_lens = reinterpret_cast<int32_t*>(t->small_out);
    } else {
      dout_lens = c.take<int32_t>(want_out_lens ? n : 0);
      Stager* sg = Stager::get(t->device);
      auto copy_in = [&](void* dst, const void* src, size_t bytes) -> int {
        if (!bytes) return PSKV_OK;
        // (buffers of the pinned pool are within reach of the copy engines as they are)
        if (sg && bytes >= kPipeBytes && !host_pool_owns(src, bytes))
          return sg->to_device(dst, src, bytes, t->stream, nullptr);
        PSKV_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, t->stream));
        return PSKV_OK;
      };
      rc = copy_in(dkeys, keys, n * 8);
      if (rc) return rc;
      if (want_lens) {
        rc = copy_in(dlens, lens, n * 4);
        if (rc) return rc;
      }
      if (sg && t->mode != PSKV_MODE_SCALAR && r.nvals * 4 >= kPipeBytes && !host_pool_owns(vals, r.nvals * 4)) {
        // the values follow piece by piece while the lookup and the row kernel are already at work
        r.vals_host = vals;
        r.pipe_in = true;
      } else {
        rc = copy_in(dvals, vals, r.nvals * 4);
        if (rc) return rc;
      }
    }
    // a large response of a row mode into ordinary memory leaves piece by piece as well, each piece
    // gathered just before it travels
    const uint64_t out_room = varlen ? out_cap : fixed_out;
    r.pipe_out = pull && !too_small && t->mode != PSKV_MODE_SCALAR && out_room * 4 >= kPipeBytes &&
                 !host_pool_owns(out, out_room * 4) && Stager::get(t->device) != nullptr;
    r.keys = dkeys;
    r.vals = dvals;
    r.lens = dlens;
    r.out_lens = want_out_lens ? dout_lens : nullptr;
    r.lazy_out = pull && varlen;
    if (small && r.lazy_out) {
      r.small_out = t->small_out + small_out_at;
      r.small_out_floats = (kSmallBytes - small_out_at) / sizeof(float);
    }
  }
  if (pull && !varlen && (host || too_small) && fixed_out) {
    if (small && !too_small && fixed_out * sizeof(float) <= kSmallBytes - small_out_at) {
      r.out = reinterpret_cast<float*>(t->small_out + small_out_at);
    } else {
      rc = grow(t, &t->stage_out, fixed_out * sizeof(float));
      if (rc) return rc;
      r.out = static_cast<float*>(t->stage_out.ptr);
    }
    r.out_cap = fixed_out;
  }

  Batch bt(1);
  bt[0].t = t;
  bt[0].r = r;
  rc = run_batch(bt, push, pull);
  r = bt[0].r;
  if (out_nvals) *out_nvals = r.out_nvals;
  // Kernels of this request may still be reading the pinned request buffer, which the next
  // host-resident request overwrites from the host: no early return without a wait.
  if (small && (rc || too_small)) (void)hipStreamSynchronize(t->stream);
  if (rc) {
    t->cache_valid = false;
    return rc;
  }
  if (too_small)
    return set_error(PSKV_ESIZE_MISMATCH, "response needs %llu floats, buffer holds %llu",
                     (unsigned long long)fixed_out, (unsigned long long)out_cap);

  if (host) {
    const bool out_pinned = pull && r.out_nvals && r.out >= reinterpret_cast<float*>(t->small_out) &&
                            r.out < reinterpret_cast<float*>(t->small_out + kSmallBytes);
    const bool lens_pinned = r.out_lens == reinterpret_cast<int32_t*>(t->small_out);
    Stager* sg = Stager::get(t->device);
    if (pull && r.out_nvals && !out_pinned) {
      if (r.gather_deferred || (sg && r.out_nvals * 4 >= kPipeBytes && !host_pool_owns(out, r.out_nvals * 4))) {
        // piece by piece: the gather of a piece (when it is still owed), its transfer, and the copy
        // into the caller's buffer overlap with those of the neighbouring pieces
        if (!sg) return set_error(PSKV_ENOMEM, "no pinned memory to stage the response through");
        std::function<int(size_t, size_t)> gather;
        if (r.gather_deferred) {
          gather = [&](size_t off, size_t len) {
            return r.gather_varlen ? launch_rows_piece<true>(bt, kOpGather, off / 4, len / 4)
                                   : launch_rows_piece<false>(bt, kOpGather, off / 4, len / 4);
          };
        }
        rc = sg->to_host(out, r.out, r.out_nvals * 4, t->stream, gather);
        if (rc) return rc;
      } else {
        PSKV_HIP(hipMemcpyAsync(out, r.out, r.out_nvals * 4, hipMemcpyDeviceToHost, t->stream));
      }
    }
    if (pull && varlen && out_lens && n && !lens_pinned)
      PSKV_HIP(hipMemcpyAsync(out_lens, r.out_lens, n * 4, hipMemcpyDeviceToHost, t->stream));
    if (small_part >= 0) {
      // no device-detected errors in this mode and nothing to hand back: the caller's buffers have
      // been copied, the kernel is queued, later requests follow it on the stream
      PSKV_HIP(hipEventRecord(t->small_done[small_part], t->stream));
      t->small_pending[small_part] = true;
      t->small_newest = small_part;
      t->small_next = (small_part + 1) % kSmallParts;
    } else if (t->mode == PSKV_MODE_SCALAR) {
      // no device-detected errors in this mode: waiting for the stream is all that is left
      PSKV_HIP(hipStreamSynchronize(t->stream));
    } else {
      rc = read_state(t);  // also waits for the copies above
      if (rc) return rc;
      rc = report_device_errors(t);
      if (rc) {
        t->cache_valid = false;
        return rc;
      }
    }
    if (out_pinned) std::memcpy(out, r.out, r.out_nvals * 4);
    if (pull && varlen && out_lens && n && lens_pinned) std::memcpy(out_lens, r.out_lens, n * 4);
  }
  return PSKV_OK;
}

// Tables that one launch can serve together: one device, one mode, one stream.
int check_group(pskv_table* const* tables, size_t S) {
  if (!tables && S) return set_error(PSKV_EINVAL, "null table list");
  for (size_t s = 0; s < S; ++s) {
    if (!tables[s]) return set_error(PSKV_EINVAL, "tables[%zu] is null", s);
    if (tables[s]->device != tables[0]->device || tables[s]->mode != tables[0]->mode)
      return set_error(PSKV_EINVAL, "tables[%zu] differs from tables[0] in device or mode", s);
    if (tables[s]->stream != tables[0]->stream)
      return set_error(PSKV_EINVAL,
                       "tables[%zu] runs on a stream of its own: create the tables of a group with "
                       "pskv_opts.stream = pskv_table_stream(first table)", s);
    for (size_t q = 0; q < s; ++q)
      if (tables[q] == tables[s]) return set_error(PSKV_EINVAL, "tables[%zu] is tables[%zu]", s, q);
  }
  return PSKV_OK;
}

// pskv_push_multi / pskv_pull_multi: slice s of the request, keys [pos[s], pos[s+1]), goes to
// tables[s]; slices without keys are skipped as KVWorker::Send skips them (kv_app.h:590-595).
int request_multi(pskv_table* const* tables, size_t S, bool push, bool pull, const uint64_t* keys,
                  const uint64_t* pos, const float* vals, const uint64_t* val_pos, const int32_t* lens,
                  float* out, const uint64_t* out_pos, int32_t* out_lens, uint64_t* out_nvals,
                  int memkind, int replay = 0) {
  clear_error();
  if (memkind != PSKV_MEM_DEVICE)
    return set_error(PSKV_EINVAL, "the multi-table entry points take device-resident buffers "
                                  "(PSKV_MEM_DEVICE); host-resident requests go table by table");
  if (out_nvals)
    for (size_t s = 0; s < S; ++s) out_nvals[s] = 0;
  if (S == 0) return PSKV_OK;
  int rc = check_group(tables, S);
  if (rc) return rc;
  if (!pos) return set_error(PSKV_EINVAL, "null pos");
  const int mode = tables[0]->mode;
  const bool varlen = mode == PSKV_MODE_VARLEN;
  if (pos[S] != pos[0] && !keys) return set_error(PSKV_EINVAL, "null keys");
  if (push && !val_pos) return set_error(PSKV_EINVAL, "null val_pos");
  if (pull && varlen && !out_pos) return set_error(PSKV_EINVAL, "a var-len pull needs out_pos");
  // everything the host can check, for every slice, before anything is enqueued
  std::vector<Request> reqs(S);
  for (size_t s = 0; s < S; ++s) {
    if (pos[s + 1] < pos[s]) return set_error(PSKV_EINVAL, "pos[%zu] > pos[%zu]", s, s + 1);
    Request& r = reqs[s];
    r = Request{};
    r.push = push;
    r.pull = pull;
    r.replay = replay;
    r.n = pos[s + 1] - pos[s];
    r.keys = keys + pos[s];
    if (push) {
      if (val_pos[s + 1] < val_pos[s]) return set_error(PSKV_EINVAL, "val_pos[%zu] > val_pos[%zu]", s, s + 1);
      r.nvals = val_pos[s + 1] - val_pos[s];
      r.vals = vals + val_pos[s];
      r.lens = (varlen && lens) ? lens + pos[s] : nullptr;
      if (r.nvals && !vals) return set_error(PSKV_EINVAL, "null vals");
    }
    if (!r.n) {
      if (r.nvals) return set_error(PSKV_ESIZE_MISMATCH, "slice %zu has values but no keys", s);
      continue;
    }
    rc = validate(tables[s], push, pull, r.n, r.nvals, r.lens, varlen && push ? r.n : 0, memkind);
    if (rc) return rc;
    if (pull) {
      const uint64_t k = mode == PSKV_MODE_SCALAR ? 1 : tables[s]->row_len;
      const uint64_t at = out_pos ? out_pos[s] : pos[s] * k;
      if (out_pos && out_pos[s + 1] < out_pos[s])
        return set_error(PSKV_EINVAL, "out_pos[%zu] > out_pos[%zu]", s, s + 1);
      r.out_cap = out_pos ? out_pos[s + 1] - out_pos[s] : r.n * k;
      r.out = out ? out + at : nullptr;
      if (!varlen) {
        if (r.out_cap < r.n * k)
          return set_error(PSKV_ESIZE_MISMATCH, "slice %zu answers %llu floats, out_pos leaves room for %llu",
                           s, (unsigned long long)(r.n * k), (unsigned long long)r.out_cap);
        if (!r.out) return set_error(PSKV_EINVAL, "null out");
      } else {
        r.out_lens = out_lens ? out_lens + pos[s] : nullptr;
        r.need_total = out_nvals != nullptr;
      }
    }
  }
  DeviceGuard guard(tables[0]->device);
  if (!guard.ok()) return set_error(PSKV_EHIP, "cannot select device %d", tables[0]->device);
  Batch bt;
  std::vector<size_t> who;
  auto flush = [&]() -> int {
    if (bt.empty()) return PSKV_OK;
    const int r = run_batch(bt, push, pull);
    for (size_t i = 0; i < bt.size(); ++i) {
      if (out_nvals) out_nvals[who[i]] = bt[i].r.out_nvals;
      if (r) bt[i].t->cache_valid = false;
    }
    bt.clear();
    who.clear();
    return r;
  };
  for (size_t s = 0; s < S; ++s) {
    if (!reqs[s].n) continue;
    Item it;
    it.t = tables[s];
    it.r = reqs[s];
    bt.push_back(it);
    who.push_back(s);
    if (bt.size() == (size_t)kMaxBatch) {
      rc = flush();
      if (rc) return rc;
    }
  }
  return flush();
}

}  // namespace

extern "C" {

int pskv_table_create(pskv_table** out, const pskv_opts* opts) {
  clear_error();
  if (!out || !opts) return set_error(PSKV_EINVAL, "null argument");
  *out = nullptr;
  if (opts->mode < PSKV_MODE_SCALAR || opts->mode > PSKV_MODE_VARLEN)
    return set_error(PSKV_EINVAL, "bad mode %d", opts->mode);
  if (opts->max_load < 0.f || opts->max_load > 0.9f)
    return set_error(PSKV_EINVAL, "max_load must lie in (0, 0.9]");
  int ndev = 0;
  if (hipGetDeviceCount(&ndev) != hipSuccess || ndev <= 0)
    return set_error(PSKV_EHIP, "no HIP device available");
  if (opts->device < 0 || opts->device >= ndev)
    return set_error(PSKV_EINVAL, "device %d out of range (%d present)", opts->device, ndev);
  DeviceGuard guard(opts->device);
  if (!guard.ok()) return set_error(PSKV_EHIP, "cannot select device %d", opts->device);

  pskv_table* t = new (std::nothrow) pskv_table();
  if (!t) return set_error(PSKV_ENOMEM, "out of host memory");
  t->device = opts->device;
  t->mode = opts->mode;
  t->max_load = opts->max_load > 0.f ? opts->max_load : 0.5f;
  t->row_len = opts->mode == PSKV_MODE_FIXED ? opts->row_len : 0;
  t->sc_min_keys = kScalarCacheMinKeys;
  if (const char* e = std::getenv("PSKV_SCALAR_CACHE_MIN_KEYS")) t->sc_min_keys = std::strtoull(e, nullptr, 10);
  auto fail = [&](int rc) {
    pskv_table_destroy(t);
    return rc;
  };
  if (opts->stream) {
    t->stream = static_cast<hipStream_t>(opts->stream);
  } else {
    if (hipStreamCreateWithFlags(&t->stream, hipStreamNonBlocking) != hipSuccess)
      return fail(set_error(PSKV_EHIP, "hipStreamCreateWithFlags failed"));
    t->own_stream = true;
  }
  const uint64_t keys = opts->initial_capacity ? opts->initial_capacity : kDefaultCapacity;
  t->cap = std::max(kMinSlots, next_pow2((uint64_t)((double)keys / t->max_load) + 1));
  int rc = alloc_slots(t->cap, &t->slots, t->stream, &t->slots_pooled);
  if (rc) return fail(rc);
  if (hipMalloc(reinterpret_cast<void**>(&t->st), sizeof(DevState)) != hipSuccess ||
      hipMemsetAsync(t->st, 0, sizeof(DevState), t->stream) != hipSuccess ||
      hipHostMalloc(reinterpret_cast<void**>(&t->st_host), sizeof(StateView), hipHostMallocCoherent) !=
          hipSuccess ||
      hipHostMalloc(reinterpret_cast<void**>(&t->snap), sizeof(Snapshot), hipHostMallocDefault) !=
          hipSuccess ||
      hipHostMalloc(reinterpret_cast<void**>(&t->outcome), sizeof(unsigned long long), hipHostMallocCoherent) !=
          hipSuccess ||
      // coherent: the GPU does not cache these two, so each request sees what the host just wrote
      hipHostMalloc(reinterpret_cast<void**>(&t->small_in), kSmallBytes, hipHostMallocCoherent) !=
          hipSuccess ||
      hipHostMalloc(reinterpret_cast<void**>(&t->small_out), kSmallBytes, hipHostMallocCoherent) !=
          hipSuccess)
    return fail(set_error(PSKV_ENOMEM, "cannot allocate table state"));
  for (int q = 0; q < kSmallParts; ++q)
    if (hipEventCreateWithFlags(&t->small_done[q], hipEventDisableTiming) != hipSuccess)
      return fail(set_error(PSKV_ENOMEM, "cannot allocate table state"));
  std::memset(t->snap, 0xFF, sizeof(Snapshot));  // names no request
  *t->outcome = 0ull;
  if (t->mode != PSKV_MODE_SCALAR && opts->arena_floats) {
    t->arena_cap = (opts->arena_floats + 1023) & ~(uint64_t)1023;
    if (alloc_for_growth(reinterpret_cast<void**>(&t->arena), t->arena_cap * sizeof(float), t->stream,
                         &t->arena_pooled) != PSKV_OK)
      return fail(set_error(PSKV_ENOMEM, "cannot allocate %llu floats of row storage",
                            (unsigned long long)t->arena_cap));
  }
  const uint64_t unset = kPayloadUnset;
  if (hipMemcpyAsync(&t->st->special_payload, &unset, sizeof(unset), hipMemcpyHostToDevice, t->stream) !=
          hipSuccess ||
      hipStreamSynchronize(t->stream) != hipSuccess)
    return fail(set_error(PSKV_EHIP, "table initialisation failed"));
  g_pools[t->device < 64 ? t->device : 63].tables.fetch_add(1);
  t->counted = true;
  *out = t;
  return PSKV_OK;
}

int pskv_table_destroy(pskv_table* t) {
  if (!t) return PSKV_OK;
  DeviceGuard guard(t->device);
  if (std::getenv("PSKV_STATS"))
    fprintf(stderr, "[pskv] table %p mode %d: %llu requests, %llu slots at the end, %llu growths (%llu without asking "
            "the device, %llu into an array allocated ahead), %llu waits for exact counters, %llu for the newest record (%.0f us), %llu counter records; host time "
            "allocating %.0f us (%.0f us on the allocating thread), releasing %.0f us\n",
            (void*)t, t->mode, (unsigned long long)t->stats.requests, (unsigned long long)t->cap,
            (unsigned long long)t->stats.growths, (unsigned long long)t->stats.growths_unasked,
            (unsigned long long)t->stats.spare_used, (unsigned long long)t->stats.waits,
            (unsigned long long)t->stats.catch_ups, t->stats.catch_up_us, (unsigned long long)t->stats.records,
            t->stats.alloc_us, t->stats.ahead_us, t->stats.release_us);
  if (t->stream) (void)hipStreamSynchronize(t->stream);
  for (int k = 0; k < PSKV_KERNEL_COUNT; ++k)
    for (const EventPair& ev : t->pending[k]) t->free_events.push_back(ev);
  for (const EventPair& ev : t->free_events) {
    (void)hipEventDestroy(ev.a);
    (void)hipEventDestroy(ev.b);
  }
  // (arrays that a growth took from the stream-ordered pool go back to it)
  if (t->slots && t->slots_pooled) {
    (void)hipFreeAsync(t->slots, t->stream);
  } else if (t->slots) {
    (void)hipFree(t->slots);
  }
  if (t->arena && t->arena_pooled) {
    (void)hipFreeAsync(t->arena, t->stream);
    t->arena = nullptr;
  }
  collect_spare(t, true);
  if (t->spare && t->spare_pooled) {
    (void)hipFreeAsync(t->spare, t->stream);
  } else if (t->spare) {
    (void)hipFree(t->spare);
  }
  if (t->slots_pooled || t->arena_pooled || t->spare_pooled) (void)hipStreamSynchronize(t->stream);
  if (t->st) (void)hipFree(t->st);
  if (t->st_host) (void)hipHostFree(t->st_host);
  if (t->snap) (void)hipHostFree(t->snap);
  if (t->outcome) (void)hipHostFree(t->outcome);
  if (t->sc_vals.ptr) (void)hipFree(t->sc_vals.ptr);
  if (t->sc_slots.ptr) (void)hipFree(t->sc_slots.ptr);
  for (int q = 0; q < kSmallParts; ++q)
    if (t->small_done[q]) (void)hipEventDestroy(t->small_done[q]);
  if (t->small_in) (void)hipHostFree(t->small_in);
  if (t->small_out) (void)hipHostFree(t->small_out);
  if (t->arena) (void)hipFree(t->arena);
  if (t->ws.ptr) (void)hipFree(t->ws.ptr);
  if (t->stage.ptr) (void)hipFree(t->stage.ptr);
  if (t->tiles.ptr) (void)hipFree(t->tiles.ptr);
  if (t->tiles_aff.ptr) (void)hipFree(t->tiles_aff.ptr);
  if (t->cache_keys.ptr) (void)hipFree(t->cache_keys.ptr);
  if (t->cache_lens.ptr) (void)hipFree(t->cache_lens.ptr);
  if (t->stage_out.ptr) (void)hipFree(t->stage_out.ptr);
  if (t->own_stream && t->stream) (void)hipStreamDestroy(t->stream);
  // the last table of a device to go takes the memory the pool has kept with it
  DevicePool& dp = g_pools[t->device < 64 ? t->device : 63];
  if (t->counted && dp.tables.fetch_sub(1) == 1 && dp.known.load(std::memory_order_acquire) == 2 && dp.pool)
    (void)hipMemPoolTrimTo(dp.pool, 0);
  delete t;
  return PSKV_OK;
}

int pskv_push(pskv_table* t, const uint64_t* keys, size_t n, const float* vals, size_t nvals,
              const int32_t* lens, size_t nlens, int memkind) {
  return request(t, true, false, keys, n, vals, nvals, lens, nlens, nullptr, 0, nullptr, nullptr,
                 memkind);
}

int pskv_pull(pskv_table* t, const uint64_t* keys, size_t n, float* out, size_t out_cap,
              int32_t* out_lens, size_t* out_nvals, int memkind) {
  return request(t, false, true, keys, n, nullptr, 0, nullptr, 0, out, out_cap, out_lens,
                 out_nvals, memkind);
}

int pskv_pushpull(pskv_table* t, const uint64_t* keys, size_t n, const float* vals, size_t nvals,
                  const int32_t* lens, size_t nlens, float* out, size_t out_cap,
                  int32_t* out_lens, size_t* out_nvals, int memkind) {
  return request(t, true, true, keys, n, vals, nvals, lens, nlens, out, out_cap, out_lens,
                 out_nvals, memkind);
}

void* pskv_table_stream(pskv_table* t) { return t ? static_cast<void*>(t->stream) : nullptr; }

int pskv_push_multi(pskv_table* const* tables, size_t S, const uint64_t* keys, const uint64_t* pos,
                    const float* vals, const uint64_t* val_pos, const int32_t* lens, int memkind) {
  return request_multi(tables, S, true, false, keys, pos, vals, val_pos, lens, nullptr, nullptr, nullptr,
                       nullptr, memkind);
}

int pskv_pushpull_multi(pskv_table* const* tables, size_t S, const uint64_t* keys, const uint64_t* pos,
                        const float* vals, const uint64_t* val_pos, const int32_t* lens, float* out,
                        const uint64_t* out_pos, int32_t* out_lens, uint64_t* out_nvals, int memkind) {
  return request_multi(tables, S, true, true, keys, pos, vals, val_pos, lens, out, out_pos, out_lens, out_nvals,
                       memkind);
}

int pskv_pull_multi(pskv_table* const* tables, size_t S, const uint64_t* keys, const uint64_t* pos,
                    float* out, const uint64_t* out_pos, int32_t* out_lens, uint64_t* out_nvals,
                    int memkind) {
  return request_multi(tables, S, false, true, keys, pos, nullptr, nullptr, nullptr, out, out_pos, out_lens,
                       out_nvals, memkind);
}

struct pskv_replay {
  std::vector<pskv_table*> tables;
  std::vector<uint64_t> gen;  // pskv_table::gen of each when the recording was made
  std::vector<SavedLaunch> launches;  // PSKV_REPLAY_LAUNCHES: made again one by one instead of as a graph
  hipGraphExec_t exec = nullptr;
  hipStream_t stream = nullptr;
  int device = 0;
};

int pskv_replay_record(pskv_replay** out, pskv_table* const* tables, size_t S, int what, const uint64_t* keys,
                       const uint64_t* pos, const float* vals, const uint64_t* val_pos, const int32_t* lens,
                       float* out_vals, const uint64_t* out_pos, int32_t* out_lens) {
  clear_error();
  if (!out) return set_error(PSKV_EINVAL, "null argument");
  *out = nullptr;
  const bool push = (what & PSKV_REPLAY_PUSH) != 0, pull = (what & PSKV_REPLAY_PULL) != 0;
  const bool as_graph = (what & PSKV_REPLAY_LAUNCHES) == 0;
  if ((!push && !pull) || (what & ~(PSKV_REPLAY_PUSH | PSKV_REPLAY_PULL | PSKV_REPLAY_LAUNCHES)))
    return set_error(PSKV_EINVAL, "what = %d names neither a push nor a pull", what);
  if (S == 0) return set_error(PSKV_EINVAL, "no tables");
  int rc = check_group(tables, S);
  if (rc) return rc;
  if (!pos || pos[S] == pos[0]) return set_error(PSKV_EINVAL, "a request without keys cannot be recorded");
  auto both = [&](int replay) -> int {
    // SCALAR: a pull of the keys just pushed is the push's own read-back, so the two go as ONE request
    // with both halves (per key the push first, kv_app.h:451-459): one comparison and one pass
    if (push && pull && tables[0]->mode == PSKV_MODE_SCALAR)
      return request_multi(tables, S, true, true, keys, pos, vals, val_pos, lens, out_vals, out_pos, out_lens,
                           nullptr, PSKV_MEM_DEVICE, replay);
    int r = PSKV_OK;
    if (push)
      r = request_multi(tables, S, true, false, keys, pos, vals, val_pos, lens, nullptr, nullptr, nullptr,
                        nullptr, PSKV_MEM_DEVICE, replay);
    if (!r && pull)
      r = request_multi(tables, S, false, true, keys, pos, nullptr, nullptr, nullptr, out_vals, out_pos, out_lens,
                        nullptr, PSKV_MEM_DEVICE, replay);
    return r;
  };
  // The request itself, the ordinary way: tables grow, buffers get their sizes, the key cache is
  // filled. What the device finds wrong with it ends the recording.
  rc = both(kReplayPrime);
  if (rc) return rc;
  rc = pskv_sync_multi(tables, S);
  if (rc) return rc;
  DeviceGuard guard(tables[0]->device);
  if (!guard.ok()) return set_error(PSKV_EHIP, "cannot select device %d", tables[0]->device);
  // (an allocation that the library's own thread is making on this stream must not land in the graph)
  for (size_t s = 0; s < S; ++s) collect_spare(tables[s], true);
  hipStream_t stream = tables[0]->stream;
  // The launches of a repeat, recorded instead of run. Relaxed: other threads of the process may
  // be allocating or waiting meanwhile, which is none of this capture's business.
  PSKV_HIP(hipStreamBeginCapture(stream, hipStreamCaptureModeRelaxed));
  std::vector<SavedLaunch> saved;
  for (size_t s = 0; s < S; ++s) tables[s]->capturing = true;
  g_recording = &saved;
  rc = both(kReplayCapture);
  g_recording = nullptr;
  for (size_t s = 0; s < S; ++s) tables[s]->capturing = false;
  hipGraph_t graph = nullptr;
  const hipError_t e = hipStreamEndCapture(stream, &graph);
  if (rc || e != hipSuccess || !graph) {
    const std::string text = rc ? std::string(pskv_last_error()) : std::string();
    if (graph) (void)hipGraphDestroy(graph);
    (void)hipGetLastError();
    for (size_t s = 0; s < S; ++s) tables[s]->cache_valid = false;
    if (rc) return set_error(rc, "%s", text.c_str());
    return set_error(PSKV_EHIP, "the stream of the tables could not be captured: %s", hipGetErrorString(e));
  }
  pskv_replay* r = new (std::nothrow) pskv_replay();
  if (!r) {
    (void)hipGraphDestroy(graph);
    return set_error(PSKV_ENOMEM, "out of host memory");
  }
  const hipError_t ei = as_graph ? hipGraphInstantiate(&r->exec, graph, nullptr, nullptr, 0) : hipSuccess;
  (void)hipGraphDestroy(graph);
  if (ei != hipSuccess) {
    delete r;
    (void)hipGetLastError();
    return set_error(PSKV_EHIP, "hipGraphInstantiate: %s", hipGetErrorString(ei));
  }
  if (!as_graph) r->launches.swap(saved);
  r->stream = stream;
  r->device = tables[0]->device;
  r->tables.assign(tables, tables + S);
  for (size_t s = 0; s < S; ++s) r->gen.push_back(tables[s]->gen);
  *out = r;
  return PSKV_OK;
}

int pskv_replay_run(pskv_replay* r) {
  clear_error();
  if (!r || (!r->exec && r->launches.empty())) return set_error(PSKV_EINVAL, "null recording");
  for (size_t s = 0; s < r->tables.size(); ++s)
    if (r->tables[s]->gen != r->gen[s])
      return set_error(PSKV_ESTALE, "tables[%zu] has served other requests since the recording was made", s);
  DeviceGuard guard(r->device);
  if (!guard.ok()) return set_error(PSKV_EHIP, "cannot select device %d", r->device);
  if (r->exec) {
    PSKV_HIP(hipGraphLaunch(r->exec, r->stream));
    return PSKV_OK;
  }
  for (const SavedLaunch& l : r->launches) hipLaunchKernelGGL(l.kernel, l.grid, dim3(kBlock), 0, r->stream, l.rb);
  PSKV_HIP(hipGetLastError());
  return PSKV_OK;
}

int pskv_replay_destroy(pskv_replay* r) {
  if (!r) return PSKV_OK;
  DeviceGuard guard(r->device);
  (void)hipStreamSynchronize(r->stream);
  if (r->exec) (void)hipGraphExecDestroy(r->exec);
  delete r;
  return PSKV_OK;
}

int pskv_sync_multi(pskv_table* const* tables, size_t S) {
  clear_error();
  if (S == 0) return PSKV_OK;
  int rc = check_group(tables, S);
  if (rc) return rc;
  DeviceGuard guard(tables[0]->device);
  int first = PSKV_OK;
  std::string first_text;
  for (size_t at = 0; at < S; at += kMaxBatch) {
    Batch bt(std::min<size_t>(S - at, kMaxBatch));
    for (size_t i = 0; i < bt.size(); ++i) bt[i].t = tables[at + i];
    rc = read_state_batch(bt);
    if (rc) return rc;
    for (Item& it : bt) {
      rc = report_device_errors(it.t);  // every table's error bits are cleared; the first is reported
      if (rc && !first) {
        first = rc;
        first_text = pskv_last_error();
      }
    }
  }
  if (first) return set_error(first, "%s", first_text.c_str());
  return PSKV_OK;
}

int pskv_sync(pskv_table* t) {
  clear_error();
  if (!t) return set_error(PSKV_EINVAL, "null table");
  DeviceGuard guard(t->device);
  int rc = read_state(t);
  if (rc) return rc;
  prepare_growth(t);  // (the counters are exact now)
  return report_device_errors(t);
}

int pskv_size(pskv_table* t, uint64_t* n_keys, uint64_t* n_vals) {
  clear_error();
  if (!t) return set_error(PSKV_EINVAL, "null table");
  DeviceGuard guard(t->device);
  int rc = read_state(t);
  if (rc) return rc;
  const uint64_t nk = t->count;  // includes key 2^64-1 when present
  if (n_keys) *n_keys = nk;
  if (n_vals) {
    if (t->mode == PSKV_MODE_SCALAR) {
      *n_vals = nk;
    } else if (t->mode == PSKV_MODE_FIXED) {
      *n_vals = nk * t->row_len;
    } else {
      unsigned long long* d_total = nullptr;
      PSKV_HIP(hipMalloc(reinterpret_cast<void**>(&d_total), sizeof(unsigned long long)));
      PSKV_HIP(hipMemsetAsync(d_total, 0, sizeof(unsigned long long), t->stream));
      k_sum_lens<<<dim3(grid_for(t->cap, kBlock, 4096)), dim3(kBlock), 0, t->stream>>>(
          t->slots, t->cap, t->st, d_total);
      unsigned long long total = 0;
      hipError_t e = hipMemcpyAsync(&total, d_total, sizeof(total), hipMemcpyDeviceToHost, t->stream);
      if (e == hipSuccess) e = hipStreamSynchronize(t->stream);
      (void)hipFree(d_total);
      PSKV_HIP(e);
      *n_vals = total;
    }
  }
  return PSKV_OK;
}

int pskv_dump(pskv_table* t, uint64_t* keys, int32_t* lens, size_t cap_keys, float* vals,
              size_t cap_vals, size_t* n_keys, size_t* n_vals) {
  clear_error();
  if (!t) return set_error(PSKV_EINVAL, "null table");
  uint64_t nk = 0, nv = 0;
  int rc = pskv_size(t, &nk, &nv);
  if (rc) return rc;
  if (n_keys) *n_keys = nk;
  if (n_vals) *n_vals = nv;
  if (nk > cap_keys || nv > cap_vals)
    return set_error(PSKV_ESIZE_MISMATCH, "dump needs room for %llu keys and %llu values",
                     (unsigned long long)nk, (unsigned long long)nv);
  if (nk == 0) return PSKV_OK;
  DeviceGuard guard(t->device);
  const uint64_t in_slots = t->count - (t->st_host->special_present ? 1 : 0);
  if (in_slots) {
    uint64_t* d_keys = nullptr;
    unsigned long long* d_counter = nullptr;
    PSKV_HIP(hipMalloc(reinterpret_cast<void**>(&d_keys), in_slots * sizeof(uint64_t)));
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&d_counter), sizeof(unsigned long long));
    if (e == hipSuccess) e = hipMemsetAsync(d_counter, 0, sizeof(unsigned long long), t->stream);
    if (e == hipSuccess) {
      k_collect_keys<<<dim3(grid_for(t->cap, kBlock, kMaxGrid)), dim3(kBlock), 0, t->stream>>>(
          t->slots, t->cap, d_keys, in_slots, d_counter);
      e = hipMemcpyAsync(keys, d_keys, in_slots * sizeof(uint64_t), hipMemcpyDeviceToHost, t->stream);
    }
    if (e == hipSuccess) e = hipStreamSynchronize(t->stream);
    (void)hipFree(d_keys);
    if (d_counter) (void)hipFree(d_counter);
    PSKV_HIP(e);
  }
  if (t->st_host->special_present) keys[in_slots] = kEmptyKey;
  std::sort(keys, keys + nk);
  // every key is present, so this pull changes nothing in the store
  size_t got = 0;
  std::vector<int32_t> tmp_lens;
  int32_t* lens_out = lens;
  if (t->mode == PSKV_MODE_VARLEN && !lens_out) {
    tmp_lens.resize(nk);
    lens_out = tmp_lens.data();
  }
  t->no_growth = true;
  rc = pskv_pull(t, keys, nk, vals, cap_vals, t->mode == PSKV_MODE_VARLEN ? lens_out : nullptr, &got,
                 PSKV_MEM_HOST);
  t->no_growth = false;
  if (rc) return rc;
  if (lens && t->mode != PSKV_MODE_VARLEN) {
    const int32_t l = t->mode == PSKV_MODE_SCALAR ? 1 : (int32_t)t->row_len;
    for (uint64_t i = 0; i < nk; ++i) lens[i] = l;
  }
  return PSKV_OK;
}

int pskv_prof_enable(pskv_table* t, int on) {
  if (!t) return set_error(PSKV_EINVAL, "null table");
  t->prof = on != 0;
  return PSKV_OK;
}

int pskv_prof_reset(pskv_table* t) {
  if (!t) return set_error(PSKV_EINVAL, "null table");
  DeviceGuard guard(t->device);
  int rc = prof_collect(t);
  for (int k = 0; k < PSKV_KERNEL_COUNT; ++k) {
    t->launches[k] = 0;
    t->total_ms[k] = 0.0;
    t->samples[k].clear();
  }
  return rc;
}

int pskv_prof_read(pskv_table* t, int kernel, uint64_t* launches, double* total_ms) {
  if (!t) return set_error(PSKV_EINVAL, "null table");
  if (kernel < 0 || kernel >= PSKV_KERNEL_COUNT) return set_error(PSKV_EINVAL, "bad kernel id");
  DeviceGuard guard(t->device);
  int rc = prof_collect(t);
  if (launches) *launches = t->launches[kernel];
  if (total_ms) *total_ms = t->total_ms[kernel];
  return rc;
}

int pskv_prof_samples(pskv_table* t, int kernel, float* out_ms, size_t cap, size_t* n) {
  if (!t || !n) return set_error(PSKV_EINVAL, "null argument");
  if (kernel < 0 || kernel >= PSKV_KERNEL_COUNT) return set_error(PSKV_EINVAL, "bad kernel id");
  DeviceGuard guard(t->device);
  int rc = prof_collect(t);
  const std::vector<float>& v = t->samples[kernel];
  *n = v.size();
  if (out_ms)
    for (size_t i = 0; i < v.size() && i < cap; ++i) out_ms[i] = v[i];
  return rc;
}

int pskv_copy_probe(pskv_table* t, void* dst, const void* src, size_t bytes) {
  if (!t) return set_error(PSKV_EINVAL, "null table");
  if ((bytes & 15) || (reinterpret_cast<uintptr_t>(dst) & 15) || (reinterpret_cast<uintptr_t>(src) & 15))
    return set_error(PSKV_EINVAL, "copy probe needs 16-byte aligned buffers and size");
  if (!bytes) return PSKV_OK;
  DeviceGuard guard(t->device);
  const uint64_t n16 = bytes / 16;
  if ((n16 + kBlock - 1) / kBlock > 0x7fffffffull) return set_error(PSKV_EINVAL, "copy too large");
  launch(t, PSKV_KERNEL_COPY, k_copy, dim3((unsigned)((n16 + kBlock - 1) / kBlock)), dim3(kBlock),
         static_cast<f32x4*>(dst), static_cast<const f32x4*>(src), n16);
  PSKV_HIP(hipGetLastError());
  return PSKV_OK;
}

int pskv_table_counters(pskv_table* t, uint64_t* out, size_t cap) {
  clear_error();
  if (!t || (!out && cap)) return set_error(PSKV_EINVAL, "null argument");
  const uint64_t v[PSKV_COUNTER_COUNT] = {t->stats.requests, t->stats.growths, t->stats.growths_unasked,
                                          t->stats.spare_used, t->stats.waits, t->stats.catch_ups,
                                          t->stats.records, t->cap};
  for (size_t i = 0; i < cap && i < (size_t)PSKV_COUNTER_COUNT; ++i) out[i] = v[i];
  return PSKV_OK;
}

int pskv_device_trim(int device) {
  clear_error();
  if (device < 0 || device >= 64) return set_error(PSKV_EINVAL, "device %d out of range", device);
  DevicePool& dp = g_pools[device];
  DeviceGuard guard(device);
  if (!guard.ok()) return set_error(PSKV_EHIP, "cannot select device %d", device);
  if (dp.known.load(std::memory_order_acquire) == 2 && dp.pool) {
    PSKV_HIP(hipDeviceSynchronize());  // what streams have freed into the pool is the pool's once they got there
    PSKV_HIP(hipMemPoolTrimTo(dp.pool, 0));
  }
  return match_trim(device);
}

const char* pskv_last_error(void) { return g_last_error.c_str(); }
const char* pskv_version(void) { return "pskv 0.1 gfx950"; }

}  // extern "C"
