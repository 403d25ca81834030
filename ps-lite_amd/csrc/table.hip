// Host side of the HBM-resident key-value store: owns the slot array, the row
// arena and the per-request workspace, sizes them, and enqueues the kernels of
// table_kernels.h in request order on one stream. This is what a ps-lite server
// calls in place of KVServerDefaultHandle (include/ps/kv_app.h:440-463).
#include <algorithm>
#include <atomic>
#include <cstring>
#include <new>
#include <string>
#include <vector>

#include <hip/hip_ext.h>

#include "host_common.h"
#include "scan.h"
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
constexpr size_t kMaxProfSamples = 65536;
constexpr uint64_t kSlackBytes = 256ull << 20;  // tables up to this size trade memory for fewer waits
// Host-resident requests up to this size (per direction) skip the copy commands: the kernels
// read the request from, and write the response to, pinned host memory mapped into the GPU.
constexpr size_t kSmallBytes = 1024u << 10;

// A device buffer that only grows. Contents are not kept across growth.
struct GrowBuf {
  void* ptr = nullptr;
  size_t bytes = 0;
};

struct EventPair {
  hipEvent_t a, b;
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

__global__ void k_read_state(const DevState* st, StateView* out) {
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

// One wavefront, launched behind the kernel of a SCALAR request when the table is close to a
// limit (the row modes let their lookup kernels write the record).
__global__ void k_publish(const DevState* st, Snapshot* out, uint64_t seq) {
  publish_snapshot(st, out, seq);
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
  uint64_t cap = 0;        // slots, a power of two
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
  GrowBuf stage;      // device copies of host-resident request buffers
  GrowBuf stage_out;  // device-side response of a host-resident or undersized pull
  bool no_growth = false;  // set while dumping: every key is known to be present

  // Row modes: the workspace keeps the row references, offsets and tile table of the last
  // request that computed them, and the key cache keeps that request's keys and lens, so a
  // request with the same keys (the usual case for a parameter server) can skip the lens
  // scan and every hash probe. The device decides whether the keys match; these fields only
  // say whether the buffers still have the shape the cached request gave them.
  GrowBuf cache_keys, cache_lens;
  bool cache_valid = false;
  uint64_t cache_n = 0, cache_nvals = 0;
  uint64_t epoch = 0;  // number of the last row-mode request

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
void launch(pskv_table* t, int prof_kernel, void (*kernel)(KArgs...), dim3 grid, dim3 block,
            Args... args) {
  if (t->prof && prof_kernel >= 0) {
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
      hipExtLaunchKernelGGL(kernel, grid, block, 0, t->stream, ev.a, ev.b, 0, static_cast<KArgs>(args)...);
      t->pending[prof_kernel].push_back(ev);
      return;
    }
  }
  hipLaunchKernelGGL(kernel, grid, block, 0, t->stream, static_cast<KArgs>(args)...);
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
  size_t want = std::max(bytes, b->bytes + b->bytes / 2);
  want = (want + 255) & ~(size_t)255;
  if (b == &t->ws || b == &t->tiles || b == &t->tiles_aff || b == &t->cache_keys ||
      b == &t->cache_lens)
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

int read_state(pskv_table* t) {
  k_read_state<<<dim3(1), dim3(64), 0, t->stream>>>(t->st, t->st_host);
  PSKV_HIP(hipGetLastError());
  PSKV_HIP(hipStreamSynchronize(t->stream));
  const uint64_t c = t->st_host->count;
  t->count = c;
  // everything enqueued so far is complete: the bounds become exact
  t->base_seq = t->seq;
  t->base_count = c;
  t->base_top = t->st_host->arena_top;
  t->pend_keys = t->pend_units = 0;
  return PSKV_OK;
}

// Turns device error bits into a status, clearing them on the device.
int report_device_errors(pskv_table* t) {
  const unsigned bits = t->st_host->error | t->st_host->req_error;
  if (!bits) return PSKV_OK;
  PSKV_HIP(hipMemsetAsync(&t->st->error, 0, 2 * sizeof(unsigned), t->stream));
  PSKV_HIP(hipStreamSynchronize(t->stream));
  if (bits & kDevErrFull) return set_error(PSKV_ENOMEM, "slot array full (internal sizing error)");
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

int alloc_slots(uint64_t cap, Slot** out, hipStream_t stream) {
  PSKV_HIP(hipMalloc(reinterpret_cast<void**>(out), cap * sizeof(Slot)));
  // all-ones bytes: key = empty marker
  PSKV_HIP(hipMemsetAsync(*out, 0xFF, cap * sizeof(Slot), stream));
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
  for (uint64_t r = t->base_seq; r <= s1; ++r) {
    t->pend_keys -= t->log_keys[r % pskv_table::kLog];
    t->pend_units -= t->log_units[r % pskv_table::kLog];
  }
  t->base_seq = s1 + 1;
  t->base_count = c;
  t->base_top = top;
}

int grow_slots(pskv_table* t, uint64_t keys_needed) {
  uint64_t want = next_pow2((uint64_t)((double)keys_needed / t->max_load) + 1);
  want = std::max(want, t->cap * 2);
  Slot* fresh = nullptr;
  int rc = alloc_slots(want, &fresh, t->stream);
  if (rc) return rc;
  launch(t, PSKV_KERNEL_REHASH, k_rehash, dim3(grid_for(t->cap, kBlock, kMaxGrid)), dim3(kBlock),
         (const Slot*)t->slots, t->cap, fresh, want - 1, t->st);
  PSKV_HIP(hipGetLastError());
  PSKV_HIP(hipStreamSynchronize(t->stream));
  PSKV_HIP(hipFree(t->slots));
  t->slots = fresh;
  t->cap = want;
  return PSKV_OK;
}

int grow_arena(pskv_table* t, uint64_t floats_needed, uint64_t live_floats) {
  uint64_t want = std::max(floats_needed, t->arena_cap + t->arena_cap / 2);
  want = (want + 1023) & ~(uint64_t)1023;
  float* fresh = nullptr;
  PSKV_HIP(hipMalloc(reinterpret_cast<void**>(&fresh), want * sizeof(float)));
  if (live_floats && t->arena) {
    PSKV_HIP(hipMemcpyAsync(fresh, t->arena, live_floats * sizeof(float), hipMemcpyDeviceToDevice,
                            t->stream));
  }
  PSKV_HIP(hipStreamSynchronize(t->stream));
  if (t->arena) PSKV_HIP(hipFree(t->arena));
  t->arena = fresh;
  t->arena_cap = want;
  return PSKV_OK;
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
// changes the counters (or launches k_publish behind it).
struct PublishReq {
  Snapshot* snap = nullptr;
  uint64_t seq = 0;
};

int reserve(pskv_table* t, uint64_t n, uint64_t units, uint64_t floats_per_unit, PublishReq* pub) {
  if (t->no_growth) return PSKV_OK;
  const double limit = (double)t->max_load * (double)t->cap;
  auto slots_short = [&]() { return (double)(t->base_count + t->pend_keys + n) > limit; };
  auto arena_short = [&]() {
    return units && (t->base_top + t->pend_units + units) * floats_per_unit > t->arena_cap;
  };
  // an ageing base is refreshed from the newest record whenever one has arrived (a host read)
  if (t->seq - t->base_seq >= (uint64_t)pskv_table::kLog / 4) adopt_snapshot(t);
  if (slots_short() || arena_short() || t->seq - t->base_seq >= (uint64_t)pskv_table::kLog - 1) {
    adopt_snapshot(t);
    if (slots_short() || arena_short() || t->seq - t->base_seq >= (uint64_t)pskv_table::kLog - 1) {
      int rc = read_state(t);  // exact counters, stream idle
      if (rc) return rc;
      // The wait happened because requests in flight had to be assumed to create all their
      // keys. Small tables get room for two more such requests, so that a caller who keeps
      // requests of this size in flight does not wait again on every one of them; for large
      // tables the wait is short next to their kernels and the memory is not.
      const uint64_t slack_n = t->cap * sizeof(Slot) <= kSlackBytes ? 2 * n : 0;
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
  const double limit_now = (double)t->max_load * (double)t->cap;
  const bool tight_slots = (double)(t->base_count + t->pend_keys + 2 * n) > limit_now;
  const bool tight_arena =
      units && (t->base_top + t->pend_units + 2 * units) * floats_per_unit > t->arena_cap;
  // (a base that merely grows old asks for a record every eighth request, not every one)
  const uint64_t age = t->seq - t->base_seq;
  const bool old_base = age >= (uint64_t)pskv_table::kLog / 4 && (age % 8 == 0 || age >= (uint64_t)pskv_table::kLog - 8);
  if (tight_slots || tight_arena || old_base) {
    pub->snap = t->snap;
    pub->seq = q;
  }
  return PSKV_OK;
}

// ---- request pipeline ------------------------------------------------------------
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
};

int run_scalar(pskv_table* t, Request& r) {
  r.out_nvals = r.pull ? r.n : 0;
  if (r.n == 0) return PSKV_OK;
  PublishReq pub;
  int rc = reserve(t, r.n, 0, 0, &pub);
  if (rc) return rc;
  const dim3 grid(grid_for(r.n, kBlock, kMaxGrid)), block(kBlock);
  const uint64_t mask = t->cap - 1;
  if (r.push && r.pull) {
    launch(t, PSKV_KERNEL_PUSH_SCALAR, k_scalar<true, true>, grid, block, t->slots, mask, t->st,
           r.keys, r.vals, r.out, r.n);
  } else if (r.push) {
    launch(t, PSKV_KERNEL_PUSH_SCALAR, k_scalar<true, false>, grid, block, t->slots, mask, t->st,
           r.keys, r.vals, (float*)nullptr, r.n);
  } else {
    launch(t, PSKV_KERNEL_PULL_SCALAR, k_scalar<false, true>, grid, block, t->slots, mask, t->st,
           r.keys, (const float*)nullptr, r.out, r.n);
  }
  if (pub.snap) k_publish<<<dim3(1), dim3(64), 0, t->stream>>>(t->st, pub.snap, pub.seq);
  PSKV_HIP(hipGetLastError());
  return PSKV_OK;
}

// Requests at least this large (4 MiB) are streamed with non-temporal accesses: between two
// requests of a busy server they do not survive in the caches anyway.
constexpr uint64_t kStreamFloats = 1u << 20;

template <bool VARLEN>
int launch_rows(pskv_table* t, int op, const RowsParams& p) {
  if (p.total == 0) return PSKV_OK;
  const uint64_t tile = VARLEN ? kRowsVarPerBlock : kTileFixed;  // request-side floats per workgroup
  const uint64_t ntiles = (p.total + tile - 1) / tile;
  if (ntiles > 0x7fffffffull) return set_error(PSKV_EINVAL, "request too large");
  const dim3 grid((unsigned)ntiles), block(kBlock);
  const bool stream = p.total >= kStreamFloats;
  if (op == kOpAcc) {
    if (stream) launch(t, PSKV_KERNEL_ROWS_ACC, k_rows<kOpAcc, VARLEN, true>, grid, block, p);
    else launch(t, PSKV_KERNEL_ROWS_ACC, k_rows<kOpAcc, VARLEN, false>, grid, block, p);
  } else {
    if (stream) launch(t, PSKV_KERNEL_ROWS_GATHER, k_rows<kOpGather, VARLEN, true>, grid, block, p);
    else launch(t, PSKV_KERNEL_ROWS_GATHER, k_rows<kOpGather, VARLEN, false>, grid, block, p);
  }
  PSKV_HIP(hipGetLastError());
  return PSKV_OK;
}

// Numbers a row-mode request and says whether the key cache has the right shape for it.
ReqTag next_tag(pskv_table* t, const Request& r) {
  ReqTag tag;
  tag.epoch = ++t->epoch;
  tag.pad = 0;
  tag.try_cache = (t->cache_valid && t->cache_n == r.n) ? 1u : 0u;
  return tag;
}

// Starts a row-mode request: numbers it and, when the key cache has the right shape, lets the
// device compare the request with the cached one. Call after every buffer the cache lives in
// has been grown for this request.
int begin_row_request(pskv_table* t, const Request& r, bool with_lens, ReqTag* tag) {
  *tag = next_tag(t, r);
  if (tag->try_cache) {
    k_same_keys<<<dim3((unsigned)((r.n + kBlock * 4 - 1) / (kBlock * 4))), dim3(kBlock), 0, t->stream>>>(
        r.keys, with_lens ? r.lens : nullptr, static_cast<const uint64_t*>(t->cache_keys.ptr),
        with_lens ? static_cast<const int32_t*>(t->cache_lens.ptr) : nullptr, r.n, t->st, *tag);
    PSKV_HIP(hipGetLastError());
  }
  return PSKV_OK;
}

int run_fixed(pskv_table* t, Request& r) {
  const uint64_t k = t->row_len;
  r.out_nvals = r.pull ? r.n * k : 0;
  if (r.n == 0) return PSKV_OK;
  PublishReq pub;
  int rc = reserve(t, r.n, r.n, k, &pub);
  if (rc) return rc;
  rc = grow(t, &t->ws, Carver::need(r.n, sizeof(uint64_t)));
  if (rc) return rc;
  rc = grow(t, &t->cache_keys, r.n * sizeof(uint64_t));
  if (rc) return rc;
  Carver c(t->ws.ptr);
  uint64_t* ref = c.take<uint64_t>(r.n);
  uint64_t* cache_keys = static_cast<uint64_t*>(t->cache_keys.ptr);
  ReqTag tag;
  rc = begin_row_request(t, r, false, &tag);
  if (rc) return rc;
  if (r.n >= kLookupLargeKeys) {
    launch(t, PSKV_KERNEL_LOOKUP, k_lookup_fixed<kLookupItemsLarge>,
           dim3(grid_for(r.n, kBlock * kLookupItemsLarge, kMaxGrid)), dim3(kBlock), t->slots,
           t->cap - 1, t->st, r.keys, r.n, ref, cache_keys, tag, pub.snap, pub.seq);
  } else {
    launch(t, PSKV_KERNEL_LOOKUP, k_lookup_fixed<1>, dim3(grid_for(r.n, kBlock, kMaxGrid)),
           dim3(kBlock), t->slots, t->cap - 1, t->st, r.keys, r.n, ref, cache_keys, tag, pub.snap,
           pub.seq);
  }
  PSKV_HIP(hipGetLastError());
  // push and pull both create absent keys, so either leaves references for all n keys behind
  t->cache_valid = true;
  t->cache_n = r.n;
  t->cache_nvals = r.n * k;
  RowsParams p{};
  p.arena = t->arena;
  p.ref = ref;
  p.st = t->st;
  p.n = r.n;
  p.total = r.n * k;
  p.k = k;
  p.tag = tag;
  if (r.push) {
    p.req = const_cast<float*>(r.vals);
    p.force_scalar = ((k & 3) || (reinterpret_cast<uintptr_t>(r.vals) & 15)) ? 1u : 0u;
    p.ignore_new = 0;
    rc = launch_rows<false>(t, kOpAcc, p);
    if (rc) return rc;
  }
  if (r.pull) {
    p.req = r.out;
    p.force_scalar = ((k & 3) || (reinterpret_cast<uintptr_t>(r.out) & 15)) ? 1u : 0u;
    p.ignore_new = r.push ? 1u : 0u;
    rc = launch_rows<false>(t, kOpGather, p);
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
// `items` per thread, the same split in every kernel of the request (the scan's
// per-workgroup totals are indexed by it).
template <typename K1, typename K4, typename... Args>
void launch_keys(pskv_table* t, int prof_kernel, uint64_t n, K1 k1, K4 k4, Args... args) {
  const dim3 grid((unsigned)scan_num_parts(n)), block(kBlock);
  if (scan_items(n) == kScanItemsLarge) {
    launch(t, prof_kernel, k4, grid, block, args...);
  } else {
    launch(t, prof_kernel, k1, grid, block, args...);
  }
}

// Pass 2 of a pull's scan: the request-side offsets of the response and the tile table for
// `floats` floats of room (the row kernel fills the other table).
int make_tile_tables(pskv_table* t, const int32_t* lens_out, const unsigned long long* part,
                     uint64_t* off, uint64_t n, uint64_t floats, RowsParams* p, const ReqTag& tag) {
  uint64_t ntiles_cap = 0;
  int rc = grow_tile_tables(t, floats, &ntiles_cap);
  if (rc) return rc;
  uint32_t* tk = static_cast<uint32_t*>(t->tiles.ptr);
  launch_keys(t, -1, n, k_var_offsets<1>, k_var_offsets<kScanItemsLarge>, lens_out, n, part, off, tk,
              ntiles_cap, (uint64_t)kTileVar, (const DevState*)t->st, tag);
  PSKV_HIP(hipGetLastError());
  p->tile_key = tk;
  p->tile_aff = static_cast<TileNote*>(t->tiles_aff.ptr);
  return PSKV_OK;
}

// Launches per var-len request: a push takes three (compare + scan pass 1; scan pass 2 +
// find-or-create + counter record; rows), a pull four (compare; stored lengths + scan pass 1;
// scan pass 2 + tile table; rows).
int run_varlen(pskv_table* t, Request& r) {
  r.out_nvals = 0;
  if (r.n == 0) return PSKV_OK;
  if (r.n > 0xfffffffeull) return set_error(PSKV_EINVAL, "too many keys in one request");
  const uint64_t nparts = scan_num_parts(r.n);
  const size_t need = Carver::need(r.n, 8) + Carver::need(r.n + 1, 8) + Carver::need(nparts, 8) +
                      Carver::need(r.n, 4);
  // Every buffer the key cache lives in is grown BEFORE the request is compared with the
  // cached one: a reallocation loses the cached contents and must rule the fast path out.
  int rc = grow(t, &t->ws, need);
  if (rc) return rc;
  rc = grow(t, &t->cache_keys, r.n * sizeof(uint64_t));
  if (rc) return rc;
  rc = grow(t, &t->cache_lens, r.n * sizeof(int32_t));
  if (rc) return rc;
  const bool async_pull = r.pull && !r.push && !r.need_total;
  const uint64_t tiles_for = r.push ? r.nvals : (async_pull ? r.out_cap : 0);
  uint64_t tiles_cap = 0;
  rc = grow_tile_tables(t, tiles_for, &tiles_cap);
  if (rc) return rc;

  Carver c(t->ws.ptr);
  uint64_t* ref = c.take<uint64_t>(r.n);
  uint64_t* off = c.take<uint64_t>(r.n + 1);
  unsigned long long* part = c.take<unsigned long long>(nparts);
  int32_t* tmp_lens = c.take<int32_t>(r.n);
  uint64_t* cache_keys = static_cast<uint64_t*>(t->cache_keys.ptr);
  int32_t* cache_lens = static_cast<int32_t*>(t->cache_lens.ptr);

  RowsParams p{};
  p.ref = ref;
  p.off = off;
  p.st = t->st;
  p.n = r.n;

  if (r.push) {
    PublishReq pub;
    // every key may round its row up to a 16-byte unit, every workgroup may pad its rows' start
    rc = reserve(t, r.n, r.nvals / 4 + r.n + kArenaPadUnits * nparts, 4, &pub);
    if (rc) return rc;
    if (t->cache_nvals != r.nvals) t->cache_valid = false;  // same lens would mean the same total
    const ReqTag tag = next_tag(t, r);
    launch_keys(t, -1, r.n, k_var_push_begin<1>, k_var_push_begin<kScanItemsLarge>, r.keys, r.lens, r.n,
                (const uint64_t*)cache_keys, (const int32_t*)cache_lens, part, t->st,
                (unsigned)PSKV_MAX_VARLEN_ROW, tag);
    PSKV_HIP(hipGetLastError());
    // pass 2 also fills the tile table of the request side (tile sizes are those of nvals; a
    // request whose lens do not add up to nvals is refused before it gets there)
    uint32_t* push_tile_key = static_cast<uint32_t*>(t->tiles.ptr);
    launch_keys(t, PSKV_KERNEL_LOOKUP, r.n, k_var_push_lookup<1>, k_var_push_lookup<kScanItemsLarge>,
                t->slots, t->cap - 1, t->st, r.keys, r.lens, r.n, r.nvals,
                (const unsigned long long*)part, off, r.nvals ? push_tile_key : (uint32_t*)nullptr,
                tiles_cap, (uint64_t)kTileVar, ref, cache_keys, cache_lens, tag, pub.snap, pub.seq);
    PSKV_HIP(hipGetLastError());
    t->cache_valid = true;  // whichever way the device decided, the cache now is this request
    t->cache_n = r.n;
    t->cache_nvals = r.nvals;
    if (r.nvals) {
      p.tile_key = push_tile_key;
      p.tile_aff = static_cast<TileNote*>(t->tiles_aff.ptr);
      p.req = const_cast<float*>(r.vals);
      p.arena = t->arena;
      p.total = r.nvals;
      p.force_scalar = (reinterpret_cast<uintptr_t>(r.vals) & 15) ? 1u : 0u;
      p.ignore_new = 0;
      p.tag = tag;
      rc = launch_rows<true>(t, kOpAcc, p);
      if (rc) return rc;
    }
  }
  if (r.pull) {
    int32_t* lens_out = r.out_lens ? r.out_lens : tmp_lens;
    if (r.push) {
      // a refused push must not be followed by its pull half
      rc = read_state(t);
      if (rc) return rc;
      rc = report_device_errors(t);
      if (rc) return rc;
    }
    // A pull with the keys of the cached push finds every key present with the cached length
    // and reuses its references; any other pull recomputes them and so ends the cache.
    ReqTag tag;
    rc = begin_row_request(t, r, false, &tag);
    if (rc) return rc;
    if (!tag.try_cache) t->cache_valid = false;
    launch_keys(t, PSKV_KERNEL_LOOKUP, r.n, k_var_pull_lookup<1>, k_var_pull_lookup<kScanItemsLarge>,
                (const Slot*)t->slots, t->cap - 1, t->st, r.keys, r.n, ref, lens_out,
                (const int32_t*)cache_lens, part, tag);
    PSKV_HIP(hipGetLastError());
    p.tag = tag;
    if (async_pull) {
      // No host round trip: the grid covers the caller's buffer, the kernels take the real
      // size from the scan, and a response that does not fit is reported by the next sync.
      if (r.out_cap) {
        if (!r.out) return set_error(PSKV_EINVAL, "null out");
        rc = make_tile_tables(t, lens_out, part, off, r.n, r.out_cap, &p, tag);
        if (rc) return rc;
        p.req = r.out;
        p.arena = t->arena;
        p.total = r.out_cap;
        p.total_on_device = 1;
        p.force_scalar = (reinterpret_cast<uintptr_t>(r.out) & 15) ? 1u : 0u;
        p.ignore_new = 1;
        rc = launch_rows<true>(t, kOpGather, p);
        if (rc) return rc;
      }
      return PSKV_OK;
    }
    rc = read_state(t);  // the response size is data dependent
    if (rc) return rc;
    if (t->st_host->same_epoch != tag.epoch) t->cache_valid = false;  // the pull recomputed the workspace
    const uint64_t total = t->st_host->scan_total;
    r.out_nvals = total;
    if (total > r.out_cap)
      return set_error(PSKV_ESIZE_MISMATCH, "response needs %llu floats, buffer holds %llu",
                       (unsigned long long)total, (unsigned long long)r.out_cap);
    if (total) {
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
      rc = make_tile_tables(t, lens_out, part, off, r.n, total, &p, tag);
      if (rc) return rc;
      p.req = r.out;
      p.arena = t->arena;
      p.total = total;
      p.force_scalar = (reinterpret_cast<uintptr_t>(r.out) & 15) ? 1u : 0u;
      p.ignore_new = 1;
      rc = launch_rows<true>(t, kOpGather, p);
      if (rc) return rc;
    }
  }
  return PSKV_OK;
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
      // every host-resident request ends with a wait, so the previous one is done with the buffers
      if (n) std::memcpy(dkeys, keys, n * 8);
      if (r.nvals) std::memcpy(dvals, vals, r.nvals * 4);
      if (want_lens && n) std::memcpy(dlens, lens, n * 4);
      small_out_at = out_lens_need;
      if (want_out_lens) dout_lens = reinterpret_cast<int32_t*>(t->small_out);
    } else {
      dout_lens = c.take<int32_t>(want_out_lens ? n : 0);
      if (n) PSKV_HIP(hipMemcpyAsync(dkeys, keys, n * 8, hipMemcpyHostToDevice, t->stream));
      if (r.nvals) PSKV_HIP(hipMemcpyAsync(dvals, vals, r.nvals * 4, hipMemcpyHostToDevice, t->stream));
      if (want_lens && n) PSKV_HIP(hipMemcpyAsync(dlens, lens, n * 4, hipMemcpyHostToDevice, t->stream));
    }
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

  switch (t->mode) {
    case PSKV_MODE_SCALAR: rc = run_scalar(t, r); break;
    case PSKV_MODE_FIXED: rc = run_fixed(t, r); break;
    default: rc = run_varlen(t, r); break;
  }
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
    if (pull && r.out_nvals && !out_pinned)
      PSKV_HIP(hipMemcpyAsync(out, r.out, r.out_nvals * 4, hipMemcpyDeviceToHost, t->stream));
    if (pull && varlen && out_lens && n && !lens_pinned)
      PSKV_HIP(hipMemcpyAsync(out_lens, r.out_lens, n * 4, hipMemcpyDeviceToHost, t->stream));
    if (t->mode == PSKV_MODE_SCALAR) {
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
  int rc = alloc_slots(t->cap, &t->slots, t->stream);
  if (rc) return fail(rc);
  if (hipMalloc(reinterpret_cast<void**>(&t->st), sizeof(DevState)) != hipSuccess ||
      hipMemsetAsync(t->st, 0, sizeof(DevState), t->stream) != hipSuccess ||
      hipHostMalloc(reinterpret_cast<void**>(&t->st_host), sizeof(StateView), hipHostMallocCoherent) !=
          hipSuccess ||
      hipHostMalloc(reinterpret_cast<void**>(&t->snap), sizeof(Snapshot), hipHostMallocDefault) !=
          hipSuccess ||
      // coherent: the GPU does not cache these two, so each request sees what the host just wrote
      hipHostMalloc(reinterpret_cast<void**>(&t->small_in), kSmallBytes, hipHostMallocCoherent) !=
          hipSuccess ||
      hipHostMalloc(reinterpret_cast<void**>(&t->small_out), kSmallBytes, hipHostMallocCoherent) !=
          hipSuccess)
    return fail(set_error(PSKV_ENOMEM, "cannot allocate table state"));
  std::memset(t->snap, 0xFF, sizeof(Snapshot));  // names no request
  if (t->mode != PSKV_MODE_SCALAR && opts->arena_floats) {
    t->arena_cap = (opts->arena_floats + 1023) & ~(uint64_t)1023;
    if (hipMalloc(reinterpret_cast<void**>(&t->arena), t->arena_cap * sizeof(float)) != hipSuccess)
      return fail(set_error(PSKV_ENOMEM, "cannot allocate %llu floats of row storage",
                            (unsigned long long)t->arena_cap));
  }
  const uint64_t unset = kPayloadUnset;
  if (hipMemcpyAsync(&t->st->special_payload, &unset, sizeof(unset), hipMemcpyHostToDevice, t->stream) !=
          hipSuccess ||
      hipStreamSynchronize(t->stream) != hipSuccess)
    return fail(set_error(PSKV_EHIP, "table initialisation failed"));
  *out = t;
  return PSKV_OK;
}

int pskv_table_destroy(pskv_table* t) {
  if (!t) return PSKV_OK;
  DeviceGuard guard(t->device);
  if (t->stream) (void)hipStreamSynchronize(t->stream);
  for (int k = 0; k < PSKV_KERNEL_COUNT; ++k)
    for (const EventPair& ev : t->pending[k]) t->free_events.push_back(ev);
  for (const EventPair& ev : t->free_events) {
    (void)hipEventDestroy(ev.a);
    (void)hipEventDestroy(ev.b);
  }
  if (t->slots) (void)hipFree(t->slots);
  if (t->st) (void)hipFree(t->st);
  if (t->st_host) (void)hipHostFree(t->st_host);
  if (t->snap) (void)hipHostFree(t->snap);
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

int pskv_sync(pskv_table* t) {
  clear_error();
  if (!t) return set_error(PSKV_EINVAL, "null table");
  DeviceGuard guard(t->device);
  int rc = read_state(t);
  if (rc) return rc;
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

const char* pskv_last_error(void) { return g_last_error.c_str(); }
const char* pskv_version(void) { return "pskv 0.1 gfx950"; }

}  // extern "C"
