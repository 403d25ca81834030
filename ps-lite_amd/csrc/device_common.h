// Shared device-side definitions of the pskv library (gfx950 only).
#ifndef PSKV_DEVICE_COMMON_H_
#define PSKV_DEVICE_COMMON_H_
#include <hip/hip_runtime.h>
#include <stdint.h>

#ifndef PSKV_TILE_VAR
#define PSKV_TILE_VAR 256
#endif

namespace pskv {

// ps::kMaxKey (include/ps/base.h:18). The stock server ranges never cover it
// (src/postoffice.cc:169-180), so it marks an empty slot; a caller that pushes it
// directly is served from one side slot kept in DevState.
constexpr uint64_t kEmptyKey = ~0ull;

// A launch serves up to kMaxBatch tables at once: blockIdx.y selects the table, blockIdx.x is the
// workgroup's number among those that serve it.
constexpr int kMaxBatch = 16;

// Row reference handed from the lookup kernel to the row kernels.
//   FIXED : low bits = row index
//   VARLEN: bits [28,63) = arena offset in 16-byte units, bits [0,28) = row length in floats
// bit 63 = the key was created by this request; all ones = key absent (var-len pull).
constexpr uint64_t kRefNew = 1ull << 63;
constexpr uint64_t kRefAbsent = ~0ull;
constexpr int kLenBits = 28;
constexpr uint64_t kLenMask = (1ull << kLenBits) - 1;

// Per-tile shortcut of the var-len row kernel. When the rows that overlap a request-side tile
// lie in the arena back to back, in request order and without padding, the whole tile maps to
// the arena with one offset: the arena position (in floats) of the tile's first float.
constexpr uint64_t kTileNotAffine = ~0ull;
// The note a var-len row kernel leaves per tile for requests that repeat its request: where in
// the arena the tile's floats lie when they form one or two unbroken pieces.
//   first  = arena offset (floats) that the tile's float 0 maps to, or kTileNotAffine
//   second = 0 for one piece; else (arena offset that float 0 would map to by the second
//            piece's distance + kTileNoteBias) << kTileSplitBits | index of the first float
//            of the second piece
struct alignas(16) TileNote {
  uint64_t first, second;
};
constexpr int kTileSplitBits = 10;
constexpr int64_t kTileNoteBias = 1 << kTileSplitBits;  // keeps the second distance non-negative

// sticky device-side error bits (DevState::error)
constexpr unsigned kDevErrLenChanged = 1u;  // var-len push: stored length differs
constexpr unsigned kDevErrFull = 2u;        // probe sequence found no free slot (host sizing bug)
constexpr unsigned kDevErrBadLen = 4u;      // negative or too long length
constexpr unsigned kDevErrSizeMismatch = 8u;  // lens do not add up to the number of values
constexpr unsigned kDevErrNoRoom = 16u;       // asynchronous var-len pull: response larger than the buffer
constexpr unsigned kDevErrDuplicate = 32u;    // the same key twice in one request (row modes)
constexpr unsigned kDevErrReplay = 64u;       // a replayed request no longer names the keys it was recorded with

// Payload of a slot that has been claimed but not filled in yet (slots start as all ones).
// No valid payload has bit 63 set.
constexpr uint64_t kPayloadUnset = ~0ull;

constexpr int kBlock = 256;             // threads per workgroup of every kernel here (4 waves)

struct __align__(16) Slot {
  uint64_t key;
  uint64_t payload;  // SCALAR: float bits in the low word; row modes: see above (without bit 63)
};

// Counters that every workgroup bumps are spread over kCountShards cache lines:
// atomics on one address are served one at a time, and a request can run thousands
// of workgroups.
constexpr int kCountShards = 32;
constexpr int kShardStride = 16;  // in 8-byte words: one shard per 128-byte line
constexpr int kTicketShards = 32;

struct alignas(32) DevState {
  // The first 32 bytes are what a row kernel needs to know about its request (ReqFacts below):
  // every wavefront reads them with one load.
  // "Same keys as the request that last filled the workspace" fast path of the row modes.
  // Every row-mode request has a number (epoch). cache_epoch is the request whose keys, lens,
  // row references, offsets and tile table the workspace and the key cache hold; bad_epoch ==
  // cache_epoch marks them unusable. same_epoch == e is the decision, reached once by the
  // compare kernel before anything else of request e runs, that e may reuse them.
  unsigned long long same_epoch;
  unsigned long long scan_total;       // grand total of the last lens scan
  unsigned int error;                  // sticky error bits of finished requests
  unsigned int req_error;              // error bits of the request in flight (follows `error`)
  unsigned int misaligned;             // OR of (len & 3) over the lens of the current request
  unsigned int req_flags;              // kReq* facts the workgroups of the kernel in flight have found
  // 32
  unsigned long long arena_top;        // FIXED: rows handed out; VARLEN: 16-byte units handed out
  unsigned long long special_payload;  // payload of key 2^64-1
  unsigned int special_present;
  unsigned int ticket_top;             // second level of the last-workgroup ticket (ticket_last)
  unsigned long long cache_epoch;
  unsigned long long bad_epoch;
  // FIXED: the request with this number was refused (it repeats a key): its row kernels change
  // no stored value and leave the rows it created as zero rows
  unsigned long long refused_epoch;
  // SCALAR key cache: the last request that changed cached values without touching the slots, and
  // the value of dirty_epoch up to which the slots have been brought up to date since
  unsigned long long dirty_epoch;
  unsigned long long clean_epoch;
  // keys held (slot array plus the side slot) = sum of the shards
  unsigned long long count_shard[kCountShards * kShardStride];
  // first level of the last-workgroup ticket: one counter per 128-byte line
  unsigned int ticket_sub[kTicketShards * 32];
};

// The head of DevState as one load.
struct ReqFacts {
  unsigned long long same_epoch, scan_total;
  unsigned int error, req_error, misaligned, req_flags;
};
static_assert(offsetof(DevState, same_epoch) == 0 && offsetof(DevState, scan_total) == 8 &&
                  offsetof(DevState, error) == 16 && offsetof(DevState, req_error) == 20 &&
                  offsetof(DevState, misaligned) == 24 && offsetof(DevState, req_flags) == 28,
              "ReqFacts mirrors the head of DevState");
typedef unsigned int u32x8 __attribute__((ext_vector_type(8)));
__device__ __forceinline__ ReqFacts load_req_facts(const DevState* st) {
  static_assert(sizeof(ReqFacts) == 32, "ReqFacts is the first 32 bytes of DevState");
  const u32x8 w = *reinterpret_cast<const u32x8*>(st);
  ReqFacts f;
  f.same_epoch = ((unsigned long long)w[1] << 32) | w[0];
  f.scan_total = ((unsigned long long)w[3] << 32) | w[2];
  f.error = w[4];
  f.req_error = w[5];
  f.misaligned = w[6];
  f.req_flags = w[7];
  return f;
}

// Facts about the request that workgroups report into DevState::req_flags.
constexpr unsigned kReqMisaligned = 3u;  // OR of (len & 3)
constexpr unsigned kReqBadLen = 4u;      // a length negative or above the maximum
constexpr unsigned kReqDiffer = 8u;      // a key or length differs from the cached request
constexpr unsigned kReqDuplicate = 16u;  // a key equals its left neighbour (requests are sorted)

// Counters of the table as they are after request `seq`, written by the device into pinned
// host memory so that the host can bound the counters without waiting for the stream.
// seq_begin == seq_end marks a consistent record.
struct Snapshot {
  volatile uint64_t seq_begin;
  volatile uint64_t count;
  volatile uint64_t arena_top;
  volatile uint64_t seq_end;
};

// What a row-mode kernel needs to know about the request it belongs to.
struct ReqTag {
  unsigned long long epoch;  // number of the request
  unsigned int try_cache;    // the host found the key cache structurally usable for this request
  // The request is a replay of a recorded one (a node of a HIP graph, launched again and again with
  // the same arguments, this number included): it is only ever served from the cache. When the
  // comparison finds other keys than the cached ones, none of its kernels changes or answers
  // anything and the table's error state says so (kDevErrReplay): the host has not sized anything
  // for keys that it has not seen.
  unsigned int replay;
};

// True when request `tag` carries exactly the keys (and lens) of the cached request, so that
// the row references, offsets and tile table still in the workspace are this request's too.
// The decision is written once, by the compare kernel that runs before the other kernels of
// the request, so every workgroup of every later kernel sees the same answer.
__device__ __forceinline__ bool cache_same(const DevState* st, const ReqTag& tag) {
  return st->same_epoch == tag.epoch;
}

// True in every kernel of a replayed request whose comparison has found other keys: the kernel
// returns at once.
__device__ __forceinline__ bool replay_blocked(const DevState* st, const ReqTag& tag) {
  return tag.replay != 0u && st->same_epoch != tag.epoch;
}

// Records an error of request `epoch`; whatever that request left in the workspace is not
// to be reused.
__device__ __forceinline__ void raise_error(DevState* st, unsigned bit, unsigned long long epoch) {
  atomicOr(&st->req_error, bit);
  st->bad_epoch = epoch;
}

// Finds the workgroup that finishes last among the `nblk` workgroups that serve one table in a
// launch (workgroups blockIdx.x = 0 .. nblk-1 of the table's row of the grid). Thread 0 of EVERY
// one of them calls it once, after the writes the last workgroup is to see; it returns true in
// exactly one of them, and that thread then sees those writes.
// What the callers hand to the last workgroup must have been written with device-scope
// atomics (atomicOr, publish_u64 below): those are performed at the memory side, past the
// per-XCD L2, so all a workgroup has to do before its ticket is wait for its own
// outstanding operations. A full release fence would write the L2 back instead, once per
// workgroup, which for a grid of 2,000 workgroups costs tens of microseconds.
// Two levels of counters, the first spread over kTicketShards cache lines, because atomics
// on one address are served one at a time (about 15 ns each).
// The counters are left at zero; kernels that use it must not overlap on one table.
__device__ __forceinline__ bool ticket_last(DevState* st, unsigned nblk) {
  // this thread's atomics and atomic stores are complete before its ticket is taken
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_waitcnt(0);
  unsigned shards = nblk;  // a small grid goes straight to the second level
  if (nblk > (unsigned)kTicketShards) {
    shards = (unsigned)kTicketShards;
    const unsigned sub = blockIdx.x % shards;
    const unsigned members = (nblk - sub + shards - 1) / shards;  // workgroups b with b % shards == sub
    unsigned* c = &st->ticket_sub[sub * 32];
    if (atomicAdd(c, 1u) != members - 1) return false;
    *c = 0;
  }
  if (atomicAdd(&st->ticket_top, 1u) != shards - 1) return false;
  st->ticket_top = 0;
  __threadfence();  // acquire, once per grid: nothing stale is left in this XCD's L2
  return true;
}

// A 64-bit value for the workgroup that ticket_last elects: stored past the L2.
__device__ __forceinline__ void publish_u64(unsigned long long* p, unsigned long long v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Adds the workgroup's total of `x` to one shard of the key counter. Every thread of
// the workgroup must call it. `red` holds kBlock/64 words of LDS.
__device__ __forceinline__ void block_count_add(DevState* st, unsigned x, unsigned* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = x;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned t = 0;
#pragma unroll
    for (int w = 0; w < kBlock / 64; ++w) t += red[w];
    if (t) atomicAdd(&st->count_shard[(blockIdx.x % kCountShards) * kShardStride], (unsigned long long)t);
  }
}

// Workgroup-wide exclusive prefix sum of `x` plus the workgroup total; every thread must
// call it. `red` holds kBlock/64 + 1 words of LDS and may be reused after the next barrier.
__device__ __forceinline__ unsigned long long block_excl_scan_u64(unsigned long long x,
                                                                  unsigned long long* red,
                                                                  unsigned long long& total) {
  unsigned long long inc = x;
  const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    unsigned long long y = __shfl_up(inc, d);
    if (lane >= (unsigned)d) inc += y;
  }
  __syncthreads();
  if (lane == 63) red[wave] = inc;
  __syncthreads();
  unsigned long long before = 0, t = 0;
#pragma unroll
  for (unsigned w = 0; w < kBlock / 64; ++w) {
    if (w < wave) before += red[w];
    t += red[w];
  }
  total = t;
  return before + inc - x;
}

typedef unsigned long long u64x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// One 128-bit read of a slot (key and payload together).
__device__ __forceinline__ u64x2 load_slot(const Slot* p) {
  return *reinterpret_cast<const u64x2*>(p);
}

// murmur3 finaliser: full avalanche, so evenly spaced keys (kMaxKey/n*i) spread out
__device__ __forceinline__ uint64_t mix64(uint64_t x) {
  x ^= x >> 33;
  x *= 0xff51afd7ed558ccdull;
  x ^= x >> 33;
  x *= 0xc4ceb9fe1a85ec53ull;
  x ^= x >> 33;
  return x;
}

// Home slot of a key in an array of mask + 1 slots (a power of two, at least 2): the TOP bits of
// the hash. A key's home in an array of G times the slots is then G * home + (a few more bits),
// so the keys of one stretch of an array are the keys of the G times longer stretch at the same
// relative place of the larger array, which lets a growth stream through both arrays instead of
// scattering every key (k_regrow).
__device__ __forceinline__ uint64_t home_slot(uint64_t key, uint64_t mask) {
  return mix64(key) >> __builtin_clzll(mask);
}

// Inclusive prefix sum over the 64 lanes of a wavefront. Every lane must call it.
__device__ __forceinline__ unsigned long long wave_incl_scan_u64(unsigned long long x) {
  const unsigned lane = __lane_id();
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    unsigned long long y = __shfl_up(x, d);
    if (lane >= (unsigned)d) x += y;
  }
  return x;
}

// Writes the table's counters to `out` (pinned host memory). Called by all 64 lanes of one
// wavefront, at a point of the stream where no kernel is changing the counters.
__device__ __forceinline__ void publish_snapshot(const DevState* st, Snapshot* out, uint64_t seq) {
  static_assert(kCountShards <= 64, "one lane per shard");
  const unsigned lane = threadIdx.x & 63;
  unsigned long long c = lane < kCountShards ? st->count_shard[lane * kShardStride] : 0ull;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o);
  if (lane != 0) return;
  out->seq_begin = seq;
  __threadfence_system();
  out->count = c;
  out->arena_top = st->arena_top;
  __threadfence_system();
  out->seq_end = seq;
}

// Finds `key` or claims an empty slot for it. Returns the address of the slot's
// payload (nullptr if the table has no free slot, which the host-side sizing
// rules out). `seen` is the payload read together with the key when the key was
// already present.
__device__ __forceinline__ uint64_t* find_or_insert(Slot* __restrict__ slots, uint64_t mask,
                                                    DevState* st, uint64_t key, bool& is_new,
                                                    uint64_t& seen) {
  is_new = false;
  seen = 0;
  if (key == kEmptyKey) {
    is_new = atomicExch(&st->special_present, 1u) == 0u;
    seen = st->special_payload;
    return reinterpret_cast<uint64_t*>(&st->special_payload);
  }
  uint64_t h = home_slot(key, mask);
  // Tries to settle the key at slot `at`, whose contents `s` were read a moment ago: 1 = found,
  // 2 = claimed, 0 = the slot belongs to another key.
  auto settle = [&](uint64_t at, const u64x2& s) -> int {
    if (s.x == key) {
      seen = s.y;
      return 1;
    }
    if (s.x == kEmptyKey) {
      unsigned long long old = atomicCAS(reinterpret_cast<unsigned long long*>(&slots[at].key),
                                         (unsigned long long)kEmptyKey, (unsigned long long)key);
      if (old == kEmptyKey) {
        is_new = true;
        return 2;
      }
      if (old == key) {  // same key twice in one request: undefined for callers, but stay sane
        seen = slots[at].payload;
        return 1;
      }
    }
    return 0;
  };
  // The home slot alone first: at the fills this table runs at, most keys are settled there, and
  // one load per lane keeps the most wavefronts in flight. A key that has to walk on asks for the
  // next three slots at once (a walk of one slot per round trip made a push a tenth slower at a
  // fill of 0.4 than at 0.1).
  {
    const u64x2 s = load_slot(&slots[h]);
    if (settle(h, s)) return &slots[h].payload;
  }
  for (uint64_t probes = 0; probes <= mask; probes += 3) {
    const uint64_t h1 = (h + 1) & mask, h2 = (h + 2) & mask, h3 = (h + 3) & mask;
    const u64x2 s1 = load_slot(&slots[h1]);
    const u64x2 s2 = load_slot(&slots[h2]);
    const u64x2 s3 = load_slot(&slots[h3]);
    if (settle(h1, s1)) return &slots[h1].payload;
    if (settle(h2, s2)) return &slots[h2].payload;
    if (settle(h3, s3)) return &slots[h3].payload;
    h = h3;
  }
  atomicOr(&st->error, kDevErrFull);
  return nullptr;
}

// Lookup without insertion. Returns false when the key is absent.
__device__ __forceinline__ bool find_only(const Slot* __restrict__ slots, uint64_t mask,
                                          const DevState* st, uint64_t key, uint64_t& payload) {
  if (key == kEmptyKey) {
    payload = st->special_payload;
    return st->special_present != 0u;
  }
  uint64_t h = home_slot(key, mask);
  for (uint64_t probes = 0; probes <= mask; ++probes) {
    const u64x2 s = load_slot(&slots[h]);
    if (s.x == key) {
      payload = s.y;
      return true;
    }
    if (s.x == kEmptyKey) return false;
    h = (h + 1) & mask;
  }
  return false;
}

}  // namespace pskv
#endif  // PSKV_DEVICE_COMMON_H_
