// Worker-side kernels: the key-range slicer that replaces KVWorker::DefaultSlicer
// (include/ps/kv_app.h:517-572) and the device-side reassembly of pulled slices
// that mirrors the callback of KVWorker::AddPullCB (kv_app.h:663-714).
#include <algorithm>
#include <chrono>
#include <cstring>
#include <limits>
#include <mutex>
#include <numeric>
#include <vector>

#include "device_common.h"
#include "host_common.h"

namespace pskv {
namespace {

// A 64-ary lower_bound by one wavefront. Each round the 64 lanes probe evenly spaced keys of
// the remaining interval, a ballot counts how many are below the target (the probes are
// sorted, so the votes are a prefix of ones) and the interval shrinks 64-fold:
// ceil(log64 n) dependent loads instead of ceil(log2 n). Every lane returns the answer.
__device__ __forceinline__ uint64_t wave_lower_bound(const uint64_t* __restrict__ keys, uint64_t n,
                                                     uint64_t target, unsigned lane) {
  uint64_t lo = 0, hi = n;  // the answer lies in [lo, hi]; keys[lo..hi) are undecided
  while (hi > lo) {
    const uint64_t len = hi - lo;
    if (len <= 64) {
      const bool below = lane < len && keys[lo + lane] < target;
      lo += __popcll(__ballot(below));
      break;
    }
    const uint64_t step = (len + 63) / 64;
    const uint64_t idx = lo + (uint64_t)(lane + 1) * step - 1;
    const bool below = idx < hi && keys[idx] < target;
    const uint64_t c = __popcll(__ballot(below));
    // probes 0..c-1 are below the target, probe c (if any) is not
    const uint64_t new_lo = lo + c * step;
    const uint64_t cap = lo + (c + 1) * step - 1;
    hi = cap < hi ? cap : hi;
    lo = new_lo < hi ? new_lo : hi;
  }
  return lo;
}

// One wavefront per search target.
__global__ __launch_bounds__(kBlock) void k_bounds(const uint64_t* __restrict__ keys, uint64_t n,
                                                  const uint64_t* __restrict__ targets,
                                                  uint64_t ntargets, uint64_t* __restrict__ lb) {
  const uint64_t w = ((uint64_t)blockIdx.x * kBlock + threadIdx.x) >> 6;
  const unsigned lane = threadIdx.x & 63;
  if (w >= ntargets) return;  // whole wavefronts leave together
  const uint64_t lo = wave_lower_bound(keys, n, targets[w], lane);
  if (lane == 0) lb[w] = lo;
}

// The word behind the S+1 positions in pinned host memory tells a host that is watching it that
// the positions of call number `done_seq` are all there (0: nobody is watching).
__device__ __forceinline__ void announce_done(uint64_t* pos_host, uint64_t S, unsigned long long done_seq) {
  if (pos_host && done_seq)
    __hip_atomic_store(reinterpret_cast<unsigned long long*>(pos_host + S + 1), done_seq, __ATOMIC_RELEASE,
                       __HIP_MEMORY_SCOPE_SYSTEM);
}

// kv_app.h:528-541: pos[0] = lower_bound(keys, ranges[0].begin); every further
// boundary is searched in the suffix that starts at the previous one, which for
// sorted keys is max(previous, lower_bound over the whole array).
// One wavefront. `pos` is device memory (read by the lens sums), `pos_host` pinned host
// memory the caller reads after the stream wait (may be null); `sums` (may be null) is
// cleared for the kernel that follows.
__global__ void k_bounds_chain(const uint64_t* __restrict__ lb, uint64_t S,
                               uint64_t* __restrict__ pos, uint64_t* __restrict__ pos_host,
                               unsigned long long* __restrict__ sums, unsigned long long done_seq) {
  if (blockIdx.x != 0) return;
  if (sums)
    for (uint64_t i = threadIdx.x; i < S; i += blockDim.x) sums[i] = 0ull;
  if (threadIdx.x != 0) return;
  uint64_t p = lb[0];
  pos[0] = p;
  if (pos_host) pos_host[0] = p;
  for (uint64_t i = 0; i < S; ++i) {
    const uint64_t e = lb[i + 1];
    p = e > p ? e : p;
    pos[i + 1] = p;
    if (pos_host) pos_host[i + 1] = p;
  }
  announce_done(pos_host, S, done_seq);
}

// Both of the above in one launch when the boundaries are few (the stock case: one per server):
// one workgroup of up to 16 wavefronts, each searching one or two boundaries, then the chain.
// The boundaries travel with the launch: no read across the host link before the search.
constexpr unsigned kFusedWaves = 16;
constexpr unsigned kFusedTargets = 2 * kFusedWaves;
struct FusedTargets {
  uint64_t v[kFusedTargets];
};
__global__ __launch_bounds__(kFusedWaves * 64) void k_bounds_fused(
    const uint64_t* __restrict__ keys, uint64_t n, FusedTargets targets, uint64_t S,
    uint64_t* __restrict__ pos, uint64_t* __restrict__ pos_host, unsigned long long* __restrict__ sums,
    unsigned long long done_seq) {
  __shared__ uint64_t s_lb[kFusedTargets];
  const unsigned lane = threadIdx.x & 63, waves = blockDim.x >> 6;
  for (unsigned w = threadIdx.x >> 6; w <= S; w += waves) {  // whole wavefronts
    const uint64_t lo = wave_lower_bound(keys, n, targets.v[w], lane);
    if (lane == 0) s_lb[w] = lo;
  }
  __syncthreads();
  if (sums)
    for (uint64_t i = threadIdx.x; i < S; i += blockDim.x) sums[i] = 0ull;
  if (threadIdx.x != 0) return;
  uint64_t p = s_lb[0];
  pos[0] = p;
  if (pos_host) pos_host[0] = p;
  for (uint64_t i = 0; i < S; ++i) {
    const uint64_t e = s_lb[i + 1];
    p = e > p ? e : p;
    pos[i + 1] = p;
    if (pos_host) pos_host[i + 1] = p;
  }
  announce_done(pos_host, S, done_seq);
}

// ---- the slicer for callers that cannot allocate ------------------------------------------
// Working memory of pskv_slice_noalloc: the lower bounds of the boundary searches followed by
// the per-slice sums of lens. It lives in the code object, so every GPU that loads the library
// holds its own copy until the process ends; host code reaches it through the address that
// hipGetSymbolAddress returns on that GPU, never through this name.
constexpr size_t kNoAllocMaxRanges = PSKV_SLICE_NOALLOC_MAX_RANGES;
constexpr size_t kNoAllocLb = kNoAllocMaxRanges + 1;            // words [0, kNoAllocLb): lower bounds
constexpr size_t kNoAllocWords = kNoAllocLb + kNoAllocMaxRanges;  // then kNoAllocMaxRanges sums
static __device__ __align__(256) unsigned long long scratch[kNoAllocWords];

// Up to kFusedTargets searches whose targets travel with the launch; the answers go to lb[].
__global__ __launch_bounds__(kFusedWaves * 64) void k_bounds_args(const uint64_t* __restrict__ keys,
                                                                 uint64_t n, FusedTargets targets,
                                                                 unsigned count,
                                                                 unsigned long long* __restrict__ lb) {
  const unsigned lane = threadIdx.x & 63, waves = blockDim.x >> 6;
  for (unsigned w = threadIdx.x >> 6; w < count; w += waves) {  // whole wavefronts
    const uint64_t lo = wave_lower_bound(keys, n, targets.v[w], lane);
    if (lane == 0) lb[w] = lo;
  }
}

// What pskv_slice does on the host once the positions and the per-slice sums are known
// (kv_app.h:540-571), by one thread, with the outputs in device memory: the `first` flags,
// the coverage check, the value offsets and their checks. `late_error` is a status the host
// already knows but which the reference raises only after the coverage check.
__global__ void k_noalloc_finish(const uint64_t* __restrict__ pos,
                                 const unsigned long long* __restrict__ sums, uint64_t S, uint64_t n,
                                 uint64_t nvals, uint64_t k, int has_lens, int late_error,
                                 uint64_t* __restrict__ val_pos, uint8_t* __restrict__ used,
                                 int32_t* __restrict__ status) {
  for (uint64_t i = threadIdx.x; i <= S; i += blockDim.x) val_pos[i] = 0;
  for (uint64_t i = threadIdx.x; i < S; i += blockDim.x) used[i] = pos[i + 1] != pos[i];  // kv_app.h:540
  __syncthreads();
  if (threadIdx.x != 0) return;
  if (pos[S] != n) {  // kv_app.h:542
    *status = PSKV_EUNCOVERED_KEY;
    return;
  }
  *status = PSKV_OK;
  if (n == 0) return;  // kv_app.h:543
  if (late_error) {    // kv_app.h:549,551
    *status = late_error;
    return;
  }
  if (!has_lens) {
    for (uint64_t i = 0; i <= S; ++i) val_pos[i] = pos[i] * k;  // kv_app.h:569
    return;
  }
  uint64_t val_begin = 0, val_end = 0;  // kv_app.h:563-567 with the CHECKs of sarray.h:249
  for (uint64_t i = 0; i < S; ++i) {
    val_pos[i] = val_begin;
    if (pos[i + 1] != pos[i]) {
      val_end += sums[i];
      if (val_end < val_begin || val_end > nvals) {
        val_pos[i + 1] = val_end;
        *status = PSKV_ESIZE_MISMATCH;
        return;
      }
      val_begin = val_end;
    }
    val_pos[i + 1] = val_end;
  }
}

// Hands the per-slice sums to the host (pinned memory).
__global__ void k_export_sums(const unsigned long long* __restrict__ sums, uint64_t S,
                              unsigned long long* __restrict__ sums_host) {
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < S;
       i += (uint64_t)gridDim.x * blockDim.x)
    sums_host[i] = sums[i];
}

// kv_app.h:565 `for (int l : kv.lens) val_end += l;` for every slice at once:
// blockIdx.y is the slice, the workgroups of a slice stride over its lens.
// Sums are taken modulo 2^64 over sign-extended lens, like size_t += int.
__global__ __launch_bounds__(kBlock) void k_segment_sums(const int32_t* __restrict__ lens,
                                                        const uint64_t* __restrict__ pos,
                                                        unsigned long long* __restrict__ sums) {
  __shared__ unsigned long long red[kBlock / 64];
  const uint64_t begin = pos[blockIdx.y], end = pos[blockIdx.y + 1];
  unsigned long long s = 0;
  const uint64_t stride = (uint64_t)gridDim.x * kBlock;
  for (uint64_t i = begin + (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < end; i += stride)
    s += (unsigned long long)(long long)lens[i];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long t = 0;
    for (int w = 0; w < kBlock / 64; ++w) t += red[w];
    if (t) atomicAdd(&sums[blockIdx.y], t);
  }
}

// First key and last key + 1 of every response (FindRange arguments, kv_app.h:671).
__global__ void k_response_ends(const uint64_t* const* __restrict__ resp_keys,
                                const uint64_t* __restrict__ resp_nkeys, uint64_t R,
                                uint64_t* __restrict__ targets) {
  const uint64_t r = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= R) return;
  targets[2 * r] = resp_keys[r][0];
  targets[2 * r + 1] = resp_keys[r][resp_nkeys[r] - 1] + 1;  // wraps to 0 for kMaxKey, as Key does
}

// One piece of a concatenation: `bytes` bytes (a multiple of 4, 4-byte aligned) from src to dst.
struct Segment {
  const char* src;
  char* dst;
  uint64_t bytes;
};

struct __attribute__((packed, aligned(4))) Words4 {
  uint32_t w[4];
};

// Copies all segments of a table (blockIdx.y = segment; the workgroups of a row stride over
// it). The destination is written with aligned 128-bit stores whatever its start: the first
// lanes move single words up to the next 16-byte boundary, and the loads that feed the
// stores may then sit on any 4-byte boundary, which global memory allows.
__global__ __launch_bounds__(kBlock) void k_concat(const Segment* __restrict__ segs) {
  const Segment sg = segs[blockIdx.y];
  if (sg.bytes == 0) return;
  uint64_t head = (16 - (reinterpret_cast<uintptr_t>(sg.dst) & 15)) & 15;  // bytes to the boundary
  if (head > sg.bytes) head = sg.bytes;
  const uint64_t body = (sg.bytes - head) / 16;  // 128-bit pieces
  const uint64_t tail_at = head + body * 16;
  const uint64_t t0 = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
  if (t0 < head / 4)
    reinterpret_cast<uint32_t*>(sg.dst)[t0] = reinterpret_cast<const uint32_t*>(sg.src)[t0];
  if (t0 < (sg.bytes - tail_at) / 4)
    reinterpret_cast<uint32_t*>(sg.dst + tail_at)[t0] =
        reinterpret_cast<const uint32_t*>(sg.src + tail_at)[t0];
  const Words4* src = reinterpret_cast<const Words4*>(sg.src + head);
  f32x4* dst = reinterpret_cast<f32x4*>(sg.dst + head);
  const uint64_t stride = (uint64_t)gridDim.x * kBlock;
  for (uint64_t i = t0; i < body; i += stride) {
    const Words4 x = src[i];
    f32x4 y;
    y.x = __uint_as_float(x.w[0]);
    y.y = __uint_as_float(x.w[1]);
    y.z = __uint_as_float(x.w[2]);
    y.w = __uint_as_float(x.w[3]);
    __builtin_nontemporal_store(y, dst + i);
  }
}

// Per-call state of the slicer. Calls may come from any thread at once
// (KVWorker::Push is thread-safe, kv_app.h:101-104), so each call takes a context
// of its own from a pool and returns it afterwards.
// Watches a word of pinned host memory for `want` for up to about 200 us; false when it did
// not show up in that time (the caller then waits for the stream as usual).
bool seen_in_time(const unsigned long long* word, unsigned long long want) {
  const auto give_up = std::chrono::steady_clock::now() + std::chrono::microseconds(200);
  for (;;) {
    for (int spin = 0; spin < 256; ++spin)
      if (__atomic_load_n(word, __ATOMIC_ACQUIRE) == want) return true;
    if (std::chrono::steady_clock::now() > give_up) return false;
  }
}

struct SliceCtx {
  unsigned long long calls = 0;  // numbers the calls whose completion the host watches for
  int device = -1;
  hipStream_t stream = nullptr;
  void* dev = nullptr;      // device scratch: targets, lower bounds, positions, sums
  size_t dev_bytes = 0;
  void* pinned = nullptr;   // pinned host memory the kernels read targets from and answer into
  size_t pinned_bytes = 0;
};

std::mutex g_pool_mu;
std::vector<SliceCtx*> g_pool;

SliceCtx* take_ctx(int device) {
  {
    std::lock_guard<std::mutex> lk(g_pool_mu);
    for (size_t i = 0; i < g_pool.size(); ++i) {
      if (g_pool[i]->device == device) {
        SliceCtx* c = g_pool[i];
        g_pool.erase(g_pool.begin() + i);
        return c;
      }
    }
  }
  SliceCtx* c = new (std::nothrow) SliceCtx();
  if (!c) return nullptr;
  c->device = device;
  if (hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking) != hipSuccess) {
    delete c;
    return nullptr;
  }
  return c;
}

void give_ctx(SliceCtx* c) {
  std::lock_guard<std::mutex> lk(g_pool_mu);
  g_pool.push_back(c);
}

// A context goes back to the pool only when nothing enqueued on its stream can still touch its
// buffers: a call that leaves early (after a failed runtime call) waits for the stream first.
struct CtxLease {
  SliceCtx* c;
  bool idle = true;  // nothing has been enqueued since the stream was last waited for
  explicit CtxLease(int device) : c(take_ctx(device)) {}
  ~CtxLease() {
    if (!c) return;
    if (!idle) (void)hipStreamSynchronize(c->stream);
    give_ctx(c);
  }
};

int ctx_reserve(SliceCtx* c, size_t dev_bytes, size_t pinned_bytes) {
  if (dev_bytes > c->dev_bytes) {
    if (c->dev) PSKV_HIP(hipFree(c->dev));
    c->dev = nullptr;
    c->dev_bytes = 0;
    PSKV_HIP(hipMalloc(&c->dev, dev_bytes));
    c->dev_bytes = dev_bytes;
  }
  if (pinned_bytes > c->pinned_bytes) {
    if (c->pinned) PSKV_HIP(hipHostFree(c->pinned));
    c->pinned = nullptr;
    c->pinned_bytes = 0;
    // coherent: never cached by the GPU, so every call sees what the host wrote for it
    PSKV_HIP(hipHostMalloc(&c->pinned, pinned_bytes, hipHostMallocCoherent));
    c->pinned_bytes = pinned_bytes;
  }
  return PSKV_OK;
}

inline size_t pad256(size_t b) { return (b + 255) & ~(size_t)255; }

int launch_bounds_search(const uint64_t* keys, uint64_t n, const uint64_t* targets, uint64_t nt,
                         uint64_t* lb, hipStream_t stream) {
  const unsigned blocks = (unsigned)((nt * 64 + kBlock - 1) / kBlock);
  k_bounds<<<dim3(blocks), dim3(kBlock), 0, stream>>>(keys, n, targets, nt, lb);
  PSKV_HIP(hipGetLastError());
  return PSKV_OK;
}

}  // namespace
}  // namespace pskv

using namespace pskv;

extern "C" {

int pskv_server_ranges(uint64_t num_servers, uint64_t* range_begin, uint64_t* range_end) {
  clear_error();
  if (num_servers == 0 || !range_begin || !range_end)
    return set_error(PSKV_EINVAL, "need at least one server and two output arrays");
  const uint64_t max_key = std::numeric_limits<uint64_t>::max();  // ps::kMaxKey, base.h:18
  for (uint64_t i = 0; i < num_servers; ++i) {
    range_begin[i] = max_key / num_servers * i;        // postoffice.cc:174
    range_end[i] = max_key / num_servers * (i + 1);    // postoffice.cc:175
  }
  return PSKV_OK;
}

int pskv_slice(int device, const uint64_t* keys, size_t n, const int32_t* lens, size_t nlens,
               size_t nvals, const uint64_t* range_begin, const uint64_t* range_end, size_t S,
               uint64_t* pos, uint64_t* val_pos, uint8_t* used, int memkind) {
  clear_error();
  if (memkind != PSKV_MEM_HOST && memkind != PSKV_MEM_DEVICE)
    return set_error(PSKV_EINVAL, "bad memkind %d", memkind);
  if (!pos || !val_pos || (S && (!used || !range_begin || !range_end)))
    return set_error(PSKV_EINVAL, "null argument");
  if (n && !keys) return set_error(PSKV_EINVAL, "null keys");
  for (size_t i = 0; i <= S; ++i) pos[i] = val_pos[i] = 0;
  for (size_t i = 0; i < S; ++i) used[i] = 0;
  // kv_app.h:533 CHECK_EQ(ranges[i-1].end(), ranges[i].begin()); it fires inside the
  // loop, before the coverage check of :542
  for (size_t i = 1; i < S; ++i) {
    if (range_end[i - 1] != range_begin[i])
      return set_error(PSKV_ERANGE_GAP, "ranges[%zu].end != ranges[%zu].begin", i - 1, i);
  }
  if (S == 0) {
    if (n) return set_error(PSKV_EUNCOVERED_KEY, "no ranges for %zu keys", n);
    return PSKV_OK;
  }
  const bool has_lens = lens != nullptr && nlens != 0;

  const bool do_sums = has_lens && nlens == n;
  if (n && do_sums && S > 65535) return set_error(PSKV_EINVAL, "more than 65535 ranges with lens");
  bool on_device = n != 0;  // (device-resident requests: searches and sums on the GPU)
  if (n && memkind == PSKV_MEM_HOST) {
    // Keys in host memory are searched where they lie: S+1 lower bounds touch (S+1) log2 n keys,
    // and shipping all n keys over the host link for that would cost milliseconds at model size
    // (and a launch and a wait at any size). This is the reference's own loop (kv_app.h:524-541).
    const uint64_t* begin = keys;
    const uint64_t* end = keys + n;
    for (size_t i = 0; i < S; ++i) {
      if (i == 0) {
        pos[0] = (uint64_t)(std::lower_bound(begin, end, range_begin[0]) - begin);
        begin += pos[0];
      }
      const size_t len = (size_t)(std::lower_bound(begin, end, range_end[i]) - begin);
      begin += len;
      pos[i + 1] = pos[i] + len;
    }
    // The lens too: one core adds them up faster (8 MB in 0.2 ms) than pageable memory crosses the
    // host link (0.28 ms for the same 8 MB, before any kernel runs): the walk of kv_app.h:563-565.
    on_device = false;
    if (do_sums) {
      for (size_t i = 0; i < S; ++i) {
        uint64_t sum = 0;
        for (uint64_t j = pos[i]; j < pos[i + 1]; ++j) sum += (uint64_t)(int64_t)lens[j];
        val_pos[i + 1] = sum;  // per-slice sums for now
      }
    }
  }

  if (on_device) {
    DeviceGuard guard(device);
    if (!guard.ok()) return set_error(PSKV_EHIP, "cannot select device %d", device);
    CtxLease lease(device);
    SliceCtx* c = lease.c;
    if (!c) return set_error(PSKV_EHIP, "cannot create a slicer context on device %d", device);
    lease.idle = false;
    // device: lb[S+1] | pos[S+1] | sums[S]      pinned: targets[S+1] | pos[S+1] | sums[S]
    const size_t arr = pad256((S + 2) * 8);  // S+1 positions and the word that says they are there
    int rc = ctx_reserve(c, 3 * arr, 3 * arr);
    if (rc) return rc;
    char* d = static_cast<char*>(c->dev);
    uint64_t* d_lb = reinterpret_cast<uint64_t*>(d);
    uint64_t* d_pos = reinterpret_cast<uint64_t*>(d + arr);
    unsigned long long* d_sums = reinterpret_cast<unsigned long long*>(d + 2 * arr);
    char* h = static_cast<char*>(c->pinned);
    uint64_t* h_targets = reinterpret_cast<uint64_t*>(h);
    uint64_t* h_pos = reinterpret_cast<uint64_t*>(h + arr);
    unsigned long long* h_sums = reinterpret_cast<unsigned long long*>(h + 2 * arr);
    const int32_t* d_lens = lens;
    h_targets[0] = range_begin[0];
    for (size_t i = 0; i < S; ++i) h_targets[i + 1] = range_end[i];
    // Without lens the positions are all this call waits for, and the kernel that writes them
    // says so in pinned memory: watching that word costs about 5 us less than a stream wait.
    const unsigned long long watch = do_sums ? 0ull : ++c->calls;
    h_pos[S + 1] = 0;  // (whatever an earlier call with other ranges left at this place)
    if (S + 1 <= kFusedTargets) {  // one launch for the boundaries when they are few
      FusedTargets ft = {};
      for (size_t i = 0; i <= S; ++i) ft.v[i] = h_targets[i];
      const unsigned waves = (unsigned)std::min<size_t>(S + 1, kFusedWaves);
      k_bounds_fused<<<dim3(1), dim3(waves * 64), 0, c->stream>>>(keys, n, ft, S, d_pos, h_pos,
                                                                 do_sums ? d_sums : nullptr, watch);
      PSKV_HIP(hipGetLastError());
    } else {
      rc = launch_bounds_search(keys, n, h_targets, S + 1, d_lb, c->stream);
      if (rc) return rc;
      k_bounds_chain<<<dim3(1), dim3(64), 0, c->stream>>>(d_lb, S, d_pos, h_pos, do_sums ? d_sums : nullptr,
                                                          watch);
      PSKV_HIP(hipGetLastError());
    }
    if (do_sums) {
      uint64_t per = n / S / (kBlock * 8) + 1;
      if (per > 1024) per = 1024;
      k_segment_sums<<<dim3((unsigned)per, (unsigned)S), dim3(kBlock), 0, c->stream>>>(d_lens, d_pos,
                                                                                      d_sums);
      PSKV_HIP(hipGetLastError());
      k_export_sums<<<dim3((unsigned)((S + 255) / 256)), dim3(256), 0, c->stream>>>(d_sums, S, h_sums);
      PSKV_HIP(hipGetLastError());
    }
    if (!watch || !seen_in_time(reinterpret_cast<unsigned long long*>(h_pos + S + 1), watch))
      PSKV_HIP(hipStreamSynchronize(c->stream));
    lease.idle = true;  // (the kernel's last act was that word)
    for (size_t i = 0; i <= S; ++i) pos[i] = h_pos[i];
    if (do_sums)
      for (size_t i = 0; i < S; ++i) val_pos[i + 1] = h_sums[i];  // per-slice sums for now
  }

  for (size_t i = 0; i < S; ++i) used[i] = pos[i + 1] != pos[i];  // kv_app.h:540
  if (pos[S] != n)  // kv_app.h:542
    return set_error(PSKV_EUNCOVERED_KEY,
                     "Check failed: (pos[n]) == (send.keys.size()): %llu keys fall in the ranges, "
                     "%zu were given", (unsigned long long)pos[S], n);
  if (n == 0) return PSKV_OK;  // kv_app.h:543

  if (!has_lens) {
    const size_t k = nvals / n;  // kv_app.h:548
    if (k * n != nvals)          // kv_app.h:549
      return set_error(PSKV_ESIZE_MISMATCH, "%zu values do not divide over %zu keys", nvals, n);
    for (size_t i = 0; i <= S; ++i) val_pos[i] = pos[i] * k;  // kv_app.h:569
    return PSKV_OK;
  }
  if (nlens != n)  // kv_app.h:551
    return set_error(PSKV_ESIZE_MISMATCH, "%zu keys but %zu lens", n, nlens);
  // kv_app.h:563-567 with the CHECKs of SArray::segment (sarray.h:249)
  uint64_t val_begin = 0, val_end = 0;
  for (size_t i = 0; i < S; ++i) {
    const uint64_t sum = val_pos[i + 1];
    val_pos[i] = val_begin;
    if (pos[i + 1] != pos[i]) {
      val_end += sum;
      if (val_end < val_begin || val_end > nvals) {
        val_pos[i + 1] = val_end;
        return set_error(PSKV_ESIZE_MISMATCH, "lens of slice %zu reach past the %zu values", i, nvals);
      }
      val_begin = val_end;
    }
    val_pos[i + 1] = val_end;
  }
  return PSKV_OK;
}

namespace {
// Device address of `scratch` on every GPU this process has used the entry point on.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
unsigned long long* g_scratch_ptr[kMaxDevices] = {nullptr};

// Called with `device` current. The first call on a device asks the runtime where that
// device's copy of the array lives; later calls read the table.
int noalloc_scratch(int device, unsigned long long** out) {
  if (device < 0 || device >= kMaxDevices) return set_error(PSKV_EINVAL, "device %d out of range", device);
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (!g_scratch_ptr[device]) {
    void* p = nullptr;
    PSKV_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return set_error(PSKV_EHIP, "no device address for the slicer's working memory");
    g_scratch_ptr[device] = static_cast<unsigned long long*>(p);
  }
  *out = g_scratch_ptr[device];
  return PSKV_OK;
}
}  // namespace

int pskv_slice_noalloc(int device, void* stream, const uint64_t* keys, size_t n, const int32_t* lens,
                       size_t nlens, size_t nvals, const uint64_t* range_begin,
                       const uint64_t* range_end, size_t S, uint64_t* pos, uint64_t* val_pos,
                       uint8_t* used, int32_t* status) {
  clear_error();
  if (!pos || !val_pos || !status || (S && (!used || !range_begin || !range_end)))
    return set_error(PSKV_EINVAL, "null argument");
  if (n && !keys) return set_error(PSKV_EINVAL, "null keys");
  if (S == 0) return set_error(PSKV_EINVAL, "pskv_slice_noalloc needs at least one range");
  if (S > kNoAllocMaxRanges)
    return set_error(PSKV_EINVAL, "pskv_slice_noalloc serves at most %zu ranges, %zu were given",
                     kNoAllocMaxRanges, S);
  for (size_t i = 1; i < S; ++i) {  // kv_app.h:533
    if (range_end[i - 1] != range_begin[i])
      return set_error(PSKV_ERANGE_GAP, "ranges[%zu].end != ranges[%zu].begin", i - 1, i);
  }
  DeviceGuard guard(device);
  if (!guard.ok()) return set_error(PSKV_EHIP, "cannot select device %d", device);
  unsigned long long* ws = nullptr;
  int rc = noalloc_scratch(device, &ws);
  if (rc) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  unsigned long long* d_lb = ws;
  unsigned long long* d_sums = ws + kNoAllocLb;

  const bool has_lens = lens != nullptr && nlens != 0;
  const bool do_sums = has_lens && nlens == n && n != 0;
  int late_error = PSKV_OK;
  uint64_t k = 0;
  if (n) {
    if (!has_lens) {
      k = nvals / n;  // kv_app.h:548-549
      if (k * n != nvals) late_error = PSKV_ESIZE_MISMATCH;
    } else if (nlens != n) {  // kv_app.h:551
      late_error = PSKV_ESIZE_MISMATCH;
    }
  }
  if (S + 1 <= kFusedTargets) {  // searches, chain and the clearing of the sums in one launch
    FusedTargets ft = {};
    ft.v[0] = range_begin[0];
    for (size_t i = 0; i < S; ++i) ft.v[i + 1] = range_end[i];
    const unsigned waves = (unsigned)std::min<size_t>(S + 1, kFusedWaves);
    k_bounds_fused<<<dim3(1), dim3(waves * 64), 0, st>>>(keys, n, ft, S, pos, (uint64_t*)nullptr, d_sums, 0ull);
    PSKV_HIP(hipGetLastError());
  } else {
    for (size_t first = 0; first <= S; first += kFusedTargets) {
      const size_t count = std::min<size_t>(S + 1 - first, kFusedTargets);
      FusedTargets ft = {};
      for (size_t j = 0; j < count; ++j) {
        const size_t i = first + j;
        ft.v[j] = i == 0 ? range_begin[0] : range_end[i - 1];
      }
      const unsigned waves = (unsigned)std::min<size_t>(count, kFusedWaves);
      k_bounds_args<<<dim3(1), dim3(waves * 64), 0, st>>>(keys, n, ft, (unsigned)count, d_lb + first);
      PSKV_HIP(hipGetLastError());
    }
    k_bounds_chain<<<dim3(1), dim3(64), 0, st>>>(reinterpret_cast<const uint64_t*>(d_lb), S, pos,
                                                (uint64_t*)nullptr, d_sums, 0ull);
    PSKV_HIP(hipGetLastError());
  }
  if (do_sums) {
    uint64_t per = n / S / (kBlock * 8) + 1;
    if (per > 1024) per = 1024;
    k_segment_sums<<<dim3((unsigned)per, (unsigned)S), dim3(kBlock), 0, st>>>(lens, pos, d_sums);
    PSKV_HIP(hipGetLastError());
  }
  k_noalloc_finish<<<dim3(1), dim3(256), 0, st>>>(pos, d_sums, S, n, nvals, k, has_lens ? 1 : 0,
                                                   late_error, val_pos, used, status);
  PSKV_HIP(hipGetLastError());
  return PSKV_OK;
}

int pskv_assemble_pull(int device, const uint64_t* req_keys, size_t n, size_t R,
                       const uint64_t* const* resp_keys, const size_t* resp_nkeys,
                       const float* const* resp_vals, const size_t* resp_nvals,
                       const int32_t* const* resp_lens, float* out, size_t out_cap,
                       int32_t* out_lens, size_t* out_nvals, int memkind) {
  clear_error();
  if (memkind != PSKV_MEM_DEVICE)
    return set_error(PSKV_EINVAL,
                     "pskv_assemble_pull concatenates device-resident slices; host-resident "
                     "slices are reassembled by KVWorker itself");
  if (out_nvals) *out_nvals = 0;
  if (R && (!resp_keys || !resp_nkeys || !resp_vals || !resp_nvals))
    return set_error(PSKV_EINVAL, "null argument");
  size_t total_key = 0, total_val = 0;
  for (size_t r = 0; r < R; ++r) {
    if (resp_nkeys[r] == 0)  // front()/back() CHECK(!empty()), sarray.h:221-222
      return set_error(PSKV_EINVAL, "response %zu has no keys", r);
    total_key += resp_nkeys[r];
    total_val += resp_nvals[r];
  }
  std::vector<uint64_t> ends(2 * R);
  if (R) {
    DeviceGuard guard(device);
    if (!guard.ok()) return set_error(PSKV_EHIP, "cannot select device %d", device);
    CtxLease lease(device);
    SliceCtx* c = lease.c;
    if (!c) return set_error(PSKV_EHIP, "cannot create a context on device %d", device);
    lease.idle = false;
    // pinned, read and written by the kernels in place:
    //   key pointers[R] | nkeys[R] | targets[2R] | lower bounds[2R] | segments[2R]
    const size_t a = pad256(R * 8), b = pad256(2 * R * 8), sg = pad256(2 * R * sizeof(Segment));
    int rc = ctx_reserve(c, 0, 2 * a + 2 * b + sg);
    if (rc) return rc;
    char* h = static_cast<char*>(c->pinned);
    const uint64_t** h_ptrs = reinterpret_cast<const uint64_t**>(h);
    uint64_t* h_nk = reinterpret_cast<uint64_t*>(h + a);
    uint64_t* h_targets = reinterpret_cast<uint64_t*>(h + 2 * a);
    uint64_t* h_lb = reinterpret_cast<uint64_t*>(h + 2 * a + b);
    Segment* h_segs = reinterpret_cast<Segment*>(h + 2 * a + 2 * b);
    for (size_t r = 0; r < R; ++r) {
      h_ptrs[r] = resp_keys[r];
      h_nk[r] = resp_nkeys[r];
    }
    k_response_ends<<<dim3((unsigned)((R + 63) / 64)), dim3(64), 0, c->stream>>>(h_ptrs, h_nk, R,
                                                                                 h_targets);
    PSKV_HIP(hipGetLastError());
    rc = launch_bounds_search(req_keys, n, h_targets, 2 * R, h_lb, c->stream);
    if (rc) return rc;
    PSKV_HIP(hipStreamSynchronize(c->stream));
    lease.idle = true;
    for (size_t r = 0; r < R; ++r) {  // kv_app.h:670-677
      const uint64_t lower = h_targets[2 * r], upper = h_targets[2 * r + 1];
      const uint64_t size = upper <= lower ? 0 : h_lb[2 * r + 1] - h_lb[2 * r];  // sarray.h:283
      if (size != resp_nkeys[r])
        return set_error(PSKV_ESIZE_MISMATCH, "unmatched keys size from one server (response %zu)", r);
      ends[2 * r] = lower;
    }
    if (total_key != n)  // kv_app.h:678
      return set_error(PSKV_ESIZE_MISMATCH, "lost some servers? %zu of %zu keys answered", total_key, n);
    if (out_nvals) *out_nvals = total_val;
    if (total_val > out_cap)  // kv_app.h:686-690
      return set_error(PSKV_ESIZE_MISMATCH, "response needs %zu floats, buffer holds %zu", total_val,
                       out_cap);
    std::vector<size_t> order(R);
    std::iota(order.begin(), order.end(), (size_t)0);
    std::sort(order.begin(), order.end(),  // kv_app.h:681-684
              [&](size_t x, size_t y) { return ends[2 * x] < ends[2 * y]; });
    // kv_app.h:701-708: one launch copies every slice to its place
    size_t voff = 0, koff = 0, nseg = 0;
    uint64_t longest = 0;
    for (size_t i = 0; i < R; ++i) {
      const size_t r = order[i];
      if (resp_nvals[r]) {
        h_segs[nseg++] = Segment{reinterpret_cast<const char*>(resp_vals[r]),
                                 reinterpret_cast<char*>(out + voff), resp_nvals[r] * sizeof(float)};
        longest = std::max<uint64_t>(longest, resp_nvals[r] * sizeof(float));
      }
      voff += resp_nvals[r];
      if (out_lens && resp_lens) {
        h_segs[nseg++] = Segment{reinterpret_cast<const char*>(resp_lens[r]),
                                 reinterpret_cast<char*>(out_lens + koff), resp_nkeys[r] * sizeof(int32_t)};
        longest = std::max<uint64_t>(longest, resp_nkeys[r] * sizeof(int32_t));
      }
      koff += resp_nkeys[r];
    }
    lease.idle = false;
    for (size_t first = 0; first < nseg; first += 65535) {  // gridDim.y holds 65535 segments
      const size_t now = std::min<size_t>(nseg - first, 65535);
      const uint64_t per = std::min<uint64_t>(longest / (16 * kBlock) + 1, 4096);
      k_concat<<<dim3((unsigned)per, (unsigned)now), dim3(kBlock), 0, c->stream>>>(h_segs + first);
      PSKV_HIP(hipGetLastError());
    }
    PSKV_HIP(hipStreamSynchronize(c->stream));
    lease.idle = true;
    return PSKV_OK;
  }
  if (total_key != n)
    return set_error(PSKV_ESIZE_MISMATCH, "lost some servers? %zu of %zu keys answered", total_key, n);
  return PSKV_OK;
}

}  // extern "C"
