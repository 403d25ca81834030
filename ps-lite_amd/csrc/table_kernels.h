// Device kernels of the HBM-resident key-value store (gfx950).
//
// They replace the body of KVServerDefaultHandle::operator()
// (include/ps/kv_app.h:442-461): `store[key] += val` becomes find-or-insert in an
// open-addressing table followed by a float add, `res.vals[i] = store[key]`
// becomes a gather. The row kernels extend the same two operations to the
// multi-float layouts of KVPairs (kv_app.h:17-31).
#ifndef PSKV_TABLE_KERNELS_H_
#define PSKV_TABLE_KERNELS_H_
#include "device_common.h"
#include "scan.h"

namespace pskv {

// What the kernels of a request need to know about ONE table's share of it. A launch carries up
// to kMaxBatch of these by value (blockIdx.y selects one), so that a request which the slicer
// has cut into per-server pieces (kv_app.h:562-612) costs one launch per step and not one per
// server; the single-table entry points launch with one of them.
struct TableReq {
  Slot* slots;
  uint64_t mask;
  DevState* st;
  const uint64_t* keys;  // n sorted unique keys
  const int32_t* lens;   // VARLEN push: n row lengths
  const float* vals;     // SCALAR push: n values
  float* out;            // SCALAR pull: n values
  uint64_t n;
  uint64_t nvals;        // VARLEN push: floats pushed
  // row modes
  float* arena;              // row storage
  uint64_t* ref;             // n row references, written by the lookup kernel
  uint64_t* off;             // VARLEN: n+1 request-side row offsets in floats
  unsigned long long* part;  // VARLEN: per-workgroup totals of the lens scan
  uint32_t* tile_key;        // VARLEN: first key of every request-side tile, ntiles+1 entries
  TileNote* tile_aff;        // VARLEN: one note per tile
  uint64_t ntiles;           // VARLEN: tiles of the request (push) / room in the tile table (pull)
  uint64_t* cache_keys;      // keys (and lens) of the request whose references the workspace holds
  int32_t* cache_lens;
  int32_t* out_lens;         // VARLEN pull: n answered lengths
  Snapshot* snap;            // where the kernel that creates the request's keys leaves the counters
  uint64_t snap_seq;
  ReqTag tag;
  // row kernels
  float* req;             // push: request values (read); pull: response values (written)
  uint64_t total;         // floats in req
  uint64_t k;             // FIXED: floats per row
  uint32_t force_scalar;  // request buffer or k not 16-byte friendly
  uint32_t ignore_new;    // pull half of a push+pull: rows created by the push half hold data
  uint32_t total_on_device;  // VARLEN pull without a host round trip: the floats to move are
                             // DevState::scan_total and `total` is the room in req
  uint32_t nblk;          // workgroups of the launch in flight that serve this table
  // SCALAR key cache (a request that repeats the cached sorted key set is served from a
  // request-ordered value array): cache_keys above, the values in `arena`, the slot numbers in
  // `tile_key`
  unsigned long long* outcome;  // pinned host word that learns how the comparison went, or null
  uint32_t cache_mode;          // kCache* below
  uint32_t tile_base;           // row kernels: the launch starts at this tile of the request (a large
                                // host-resident request is served piece by piece as it arrives)
};
constexpr uint32_t kCacheOff = 0;     // SCALAR: the request neither uses nor fills the key cache
constexpr uint32_t kCacheOn = 1;      // SCALAR: serve from the cache when the keys match, else refill it
constexpr uint32_t kCachePerKey = 3;  // SCALAR pull, slots up to date: every key that sits at its cached
                                      // position is answered from the cache, the others through the slots
constexpr uint32_t kFlushUnlessSame = 1;  // k_scalar_flush: skip when the request in flight repeats the cache
constexpr uint32_t kFlushAlways = 2;
constexpr uint32_t kSlotSpecial = 0xffffffffu;  // cached slot number of key 2^64-1 (the side slot)
struct ReqBatch {
  TableReq t[kMaxBatch];
};
static_assert(sizeof(ReqBatch) <= 3840, "kernel arguments are limited to 4 KiB");

// ---------------------------------------------------------------------------------
// SCALAR mode: one float per key, kept in the low word of the slot payload so that a
// probe reads key and value with one 128-bit load.
// One lane per key. Keys are unique within a request (kv_app.h:17), so the value word of a
// slot is only ever touched by the lane that owns the key: no atomics on values, and the
// per-key sum order is the request order (requests are serialised on one stream).
// The reference's handle is a plain loop over the request (kv_app.h:451-459), so even a
// sorted request that repeats a key has a defined result there; it has the same result
// here: the lane of the first occurrence serves the whole run in order, the other lanes of
// the run stand back. Whether a lane starts or continues a run is read off the neighbouring
// lanes' keys (a shuffle; only the first and the last lane of a wavefront look at memory), which
// costs requests without repeats about 1 % of a push + pull step. One lane walks its run element
// by element, so this is for the odd repeat, not a reduction of long runs. An UNSORTED request
// that repeats a key remains a caller error with an unspecified sum.
// ---------------------------------------------------------------------------------
// Stable key sets (the idea of the reference's unused sorted-merge helper,
// include/ps/internal/parallel_kv_match.h:29-120: when both sides are sorted the same way no
// lookup is needed). The CACHE variant serves a request that repeats the cached sorted key set
// from a request-ordered value array: `cache_vals[i] += vals[i]`, fully coalesced, 12 bytes per
// key instead of a 128-byte line per probe; the slots are brought up to date (k_scalar_flush)
// before anything else looks at them. A request that does not repeat the cache goes the usual
// way and leaves its keys, their values and their slot numbers behind as the new cache.
// A pull that comes right behind the push that filled the cache (the slots are up to date then)
// needs no decision for the whole request: kCachePerKey compares key by key, in the same pass.
template <bool PUSH, bool PULL, bool CACHE>
__global__ __launch_bounds__(kBlock) void k_scalar(ReqBatch b) {
  const TableReq& d = b.t[blockIdx.y];
  const uint64_t n = d.n;
  const unsigned nblk = d.nblk;  // (the grid is sized for the table with the most workgroups)
  if (blockIdx.x >= nblk) return;
  Slot* __restrict__ slots = d.slots;
  const uint64_t mask = d.mask;
  DevState* st = d.st;
  const uint64_t* __restrict__ keys = d.keys;
  const float* __restrict__ vals = d.vals;
  float* __restrict__ out = d.out;
  const bool record = CACHE && d.cache_mode == kCacheOn;
  if (CACHE && replay_blocked(st, d.tag)) return;
  if (record && cache_same(st, d.tag)) {
    // the keys are those of the cached request: position i of the request is position i of the cache
    float* __restrict__ cv = d.arena;
    if (PUSH && blockIdx.x == 0 && threadIdx.x == 0) st->dirty_epoch = d.tag.epoch;  // the slots fall behind
    const bool vec = ((reinterpret_cast<uintptr_t>(vals) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    const uint64_t stride = (uint64_t)nblk * kBlock * 4;
    for (uint64_t i = ((uint64_t)blockIdx.x * kBlock + threadIdx.x) * 4; i < n; i += stride) {
      if (vec && i + 4 <= n) {
        f32x4 cur = *reinterpret_cast<const f32x4*>(cv + i);
        if (PUSH) cur = cur + __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(vals + i));
        if (PULL) __builtin_nontemporal_store(cur, reinterpret_cast<f32x4*>(out + i));
        if (PUSH) *reinterpret_cast<f32x4*>(cv + i) = cur;
      } else {
        for (uint64_t j = i; j < n && j < i + 4; ++j) {
          float cur = cv[j];
          if (PUSH) cur = cur + vals[j];
          if (PULL) out[j] = cur;
          if (PUSH) cv[j] = cur;
        }
      }
    }
    // (no key is created on this path: the counters are what they were)
    if (d.snap && blockIdx.x == 0 && threadIdx.x < 64) publish_snapshot(st, d.snap, d.snap_seq);
    return;
  }
  if (record && blockIdx.x == 0 && threadIdx.x == 0) st->cache_epoch = d.tag.epoch;
  constexpr bool kPerKey = CACHE && PULL && !PUSH;
  bool per_key = false, differs = false;
  if (kPerKey) {
    // (nothing writes these two words while a pull of this kind runs)
    per_key = d.cache_mode == kCachePerKey && st->cache_epoch != 0ull && st->bad_epoch != st->cache_epoch;
  }
  __shared__ unsigned red[kBlock / 64];
  unsigned created = 0;
  if (kPerKey && per_key) {
    // Four keys per lane, 128 bits per load. The cached request had no repeats, so four keys that
    // equal their cached neighbours are four different keys; the key behind them says whether
    // the last of them starts a run, which goes through the slots as a whole.
    const uint64_t* __restrict__ ck = d.cache_keys;
    const float* __restrict__ cv = d.arena;
    const bool kvec = (reinterpret_cast<uintptr_t>(keys) & 15) == 0;
    const bool ovec = (reinterpret_cast<uintptr_t>(out) & 15) == 0;
    const uint64_t stride4 = (uint64_t)nblk * kBlock * 4;
    for (uint64_t i = ((uint64_t)blockIdx.x * kBlock + threadIdx.x) * 4; i < n; i += stride4) {
      if (i + 4 <= n) {
        u64x2 x0, x1;
        if (kvec) {
          x0 = __builtin_nontemporal_load(reinterpret_cast<const u64x2*>(keys + i));
          x1 = __builtin_nontemporal_load(reinterpret_cast<const u64x2*>(keys + i + 2));
        } else {
          x0.x = keys[i], x0.y = keys[i + 1], x1.x = keys[i + 2], x1.y = keys[i + 3];
        }
        const u64x2 y0 = *reinterpret_cast<const u64x2*>(ck + i);
        const u64x2 y1 = *reinterpret_cast<const u64x2*>(ck + i + 2);
        const f32x4 v4 = *reinterpret_cast<const f32x4*>(cv + i);
        const uint64_t behind = i + 4 < n ? keys[i + 4] : ~x1.y;
        if (x0.x == y0.x && x0.y == y0.y && x1.x == y1.x && x1.y == y1.y && behind != x1.y) {
          if (ovec) {
            __builtin_nontemporal_store(v4, reinterpret_cast<f32x4*>(out + i));
          } else {
            out[i] = v4.x, out[i + 1] = v4.y, out[i + 2] = v4.z, out[i + 3] = v4.w;
          }
          continue;
        }
      }
      for (uint64_t j = i; j < n && j < i + 4; ++j) {  // key by key
        const uint64_t key = keys[j];
        if (j > 0 && keys[j - 1] == key) continue;  // inside a run: its first key answers for it
        const bool run = j + 1 < n && keys[j + 1] == key;
        if (!run && ck[j] == key) {
          out[j] = cv[j];
          continue;
        }
        differs = true;
        bool is_new;
        uint64_t seen;
        uint64_t* p = find_or_insert(slots, mask, st, key, is_new, seen);
        if (!p) continue;
        const float cur = is_new ? 0.0f : __uint_as_float((unsigned)seen);
        out[j] = cur;
        for (uint64_t r = j + 1; r < n && keys[r] == key; ++r) out[r] = cur;
        if (is_new) *reinterpret_cast<float*>(p) = cur;
        created += is_new ? 1u : 0u;
      }
    }
  }
  // every other request: one key per lane and turn through the slots
  const uint64_t n_turns = (kPerKey && per_key) ? 0 : n;
  const uint64_t stride = (uint64_t)nblk * kBlock;
  const unsigned lane = threadIdx.x & 63;
  // whole wavefronts stay in the loop together: the shuffles below need every lane
  for (uint64_t first = (uint64_t)blockIdx.x * kBlock; first < n_turns; first += stride) {
    const uint64_t i = first + threadIdx.x;
    const bool live = i < n;
    const uint64_t key = live ? keys[i] : 0;
    uint64_t before = __shfl_up(key, 1);
    uint64_t after = __shfl_down(key, 1);
    // the first and the last lane look just outside the wavefront's 64 keys; their neighbours have
    // fetched those lines already
    if (lane == 0) before = (live && i > 0) ? keys[i - 1] : ~key;
    if (lane == 63) after = (i + 1 < n) ? keys[i + 1] : ~key;
    if (!live || (i > 0 && before == key)) continue;  // past the end, or inside a run
    const bool run = i + 1 < n && after == key;
    float v = 0.0f;
    if (PUSH) v = vals[i];
    bool is_new;
    uint64_t seen;
    uint64_t* p = find_or_insert(slots, mask, st, key, is_new, seen);
    if (record && (!p || run)) st->bad_epoch = d.tag.epoch;  // not a request the cache can stand for
    if (!p) continue;
    // an absent key starts from Val() == 0, then `+=` (kv_app.h:454): 0.0f + v, not a copy
    float cur = is_new ? 0.0f : __uint_as_float((unsigned)seen);
    if (PUSH) cur = cur + v;
    if (PULL) out[i] = cur;
    if (run) {  // the rest of the run, element by element like the reference's loop
      for (uint64_t j = i + 1; j < n && keys[j] == key; ++j) {
        if (PUSH) cur = cur + vals[j];
        if (PULL) out[j] = cur;
      }
    }
    if (PUSH || is_new) *reinterpret_cast<float*>(p) = cur;
    created += is_new ? 1u : 0u;
    if (record) {
      d.cache_keys[i] = key;
      d.arena[i] = cur;
      d.tile_key[i] = key == kEmptyKey ? kSlotSpecial
                                       : (uint32_t)((reinterpret_cast<Slot*>(p - 1) - slots));
    }
  }
  block_count_add(st, created, red);
  // The workgroup that finishes last tells the host, which never waits for either, whether every
  // key of a key-by-key pull sat at its cached position and, when the host asked for it (the
  // table is close to a limit), what the counters are after this request.
  const bool want_outcome = kPerKey && d.cache_mode == kCachePerKey;
  if (want_outcome || d.snap) {
    __shared__ unsigned s_last;
    const int any = want_outcome ? __syncthreads_or(differs ? 1 : 0) : 0;
    if (threadIdx.x == 0) {
      if (any) atomicOr(&st->req_flags, kReqDiffer);
      s_last = ticket_last(st, nblk) ? 1u : 0u;
    }
    __syncthreads();
    if (!s_last) return;
    if (want_outcome && threadIdx.x == 0) {
      const bool all = (atomicExch(&st->req_flags, 0u) & kReqDiffer) == 0u && per_key;
      if (d.outcome) *d.outcome = (d.tag.epoch << 1) | (all ? 1ull : 0ull);
    }
    if (d.snap && threadIdx.x < 64) publish_snapshot(st, d.snap, d.snap_seq);
  }
}

// Writes the cached values back to their slots. Launched before anything reads or changes the
// slots of a table whose cache may be ahead of them: a request that does not repeat the cached
// keys (kFlushUnlessSame: the comparison of that request has run), a growth, a dump.
__global__ __launch_bounds__(kBlock) void k_scalar_flush(ReqBatch b) {
  const TableReq& d = b.t[blockIdx.y];
  if (blockIdx.x >= d.nblk) return;
  // nothing changes these two while this kernel runs except its own last workgroup, which writes
  // after every workgroup has read them
  const unsigned long long dirty = d.st->dirty_epoch;
  if (dirty <= d.st->clean_epoch) return;  // the slots are up to date
  if (d.cache_mode == kFlushUnlessSame && (cache_same(d.st, d.tag) || d.tag.replay)) return;
  __shared__ unsigned s_last;
  const uint64_t stride = (uint64_t)d.nblk * kBlock;
  for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < d.n; i += stride) {
    const uint32_t slot = d.tile_key[i];
    const float v = d.arena[i];
    float* dst = slot == kSlotSpecial ? reinterpret_cast<float*>(&d.st->special_payload)
                                      : reinterpret_cast<float*>(&d.slots[slot].payload);
    *dst = v;
  }
  if (threadIdx.x == 0) s_last = ticket_last(d.st, d.nblk) ? 1u : 0u;
  __syncthreads();
  if (s_last && threadIdx.x == 0) d.st->clean_epoch = dirty;
}

// ---------------------------------------------------------------------------------
// Row modes, step 1: key -> row reference.
// ---------------------------------------------------------------------------------

// The decision about a request that may repeat the cached one, taken by one thread after
// every workgroup has compared its share (`different`: any of them found a difference). If
// the decision is "different" (or the cache was not usable, or not even tried), the request
// is going to refill the cache, so it becomes the cached request right here. Epochs start
// at 1.
__device__ __forceinline__ void decide_same(DevState* st, const ReqTag& tag, bool different,
                                            unsigned long long* outcome = nullptr) {
  const bool usable =
      tag.try_cache && st->cache_epoch != 0ull && st->bad_epoch != st->cache_epoch;
  const bool same = !different && usable;
  if (tag.replay && !same) {
    // (an earlier replay of this very request may have left its number here)
    st->same_epoch = 0ull;
    atomicOr(&st->error, kDevErrReplay);
    return;
  }
  if (same) {
    st->same_epoch = tag.epoch;
  } else {
    st->cache_epoch = tag.epoch;
  }
  // the host reads this when it gets to it (never waits for it): epoch << 1 | same; only a
  // request that was in fact compared reports
  if (outcome && tag.try_cache) *outcome = (tag.epoch << 1) | (same ? 1ull : 0ull);
}

// Compares the keys of a request with the cached ones and reaches the decision for the whole
// request: the workgroup that finishes last sees whether any workgroup found a difference and
// writes same_epoch. (A var-len push, whose lens count as well, compares in k_var_push_begin.)
constexpr int kSameKeysItems = 4;
__global__ __launch_bounds__(kBlock) void k_same_keys(ReqBatch b) {
  const TableReq& d = b.t[blockIdx.y];
  if (blockIdx.x >= d.nblk) return;  // tables that have nothing to compare have no workgroups
  const uint64_t* __restrict__ keys = d.keys;
  const uint64_t* __restrict__ cache_keys = d.cache_keys;
  const uint64_t n = d.n;
  DevState* st = d.st;
  const ReqTag tag = d.tag;
  __shared__ unsigned s_last;
  constexpr int kItems = kSameKeysItems;
  static_assert(kItems % 2 == 0, "two keys per 128-bit load");
  const uint64_t base = ((uint64_t)blockIdx.x * kBlock + threadIdx.x) * kItems;
  // all loads first, then the compares; 128 bits per load where the buffers allow it (the cached
  // keys always do), the request side read past the caches
  uint64_t a[kItems], c[kItems];
  const bool vec = (reinterpret_cast<uintptr_t>(keys) & 15) == 0 && base + kItems <= n;
  if (vec) {
#pragma unroll
    for (int j = 0; j < kItems; j += 2) {
      const u64x2 x = __builtin_nontemporal_load(reinterpret_cast<const u64x2*>(keys + base + j));
      const u64x2 y = *reinterpret_cast<const u64x2*>(cache_keys + base + j);
      a[j] = x.x, a[j + 1] = x.y;
      c[j] = y.x, c[j + 1] = y.y;
    }
  } else {
#pragma unroll
    for (int j = 0; j < kItems; ++j) {
      const bool in = base + j < n;
      a[j] = in ? keys[base + j] : 0;
      c[j] = in ? cache_keys[base + j] : 0;
    }
  }
  bool differ = false;
#pragma unroll
  for (int j = 0; j < kItems; ++j) differ |= a[j] != c[j];
  const int any = __syncthreads_or(differ ? 1 : 0);
  if (threadIdx.x == 0) {
    if (any) atomicOr(&st->req_flags, kReqDiffer);
    s_last = ticket_last(st, d.nblk) ? 1u : 0u;
  }
  __syncthreads();
  if (!s_last) return;
  if (threadIdx.x == 0)
    decide_same(st, tag, (atomicExch(&st->req_flags, 0u) & kReqDiffer) != 0u, d.outcome);
}

// The counter record of a request, written by the kernel that creates its keys once every
// workgroup has taken its rows (or at once when the request creates nothing): the record then
// holds the counters as they are AFTER the request. Every thread of the workgroup calls it;
// `s_last` is one word of LDS.
__device__ __forceinline__ void publish_after_lookup(DevState* st, Snapshot* snap, uint64_t seq,
                                                     unsigned nblk, unsigned* s_last) {
  if (!snap) return;
  if (threadIdx.x == 0) *s_last = ticket_last(st, nblk) ? 1u : 0u;
  __syncthreads();
  if (*s_last && threadIdx.x < 64) publish_snapshot(st, snap, seq);
}

// Keys per thread and round of the creating lookups: 4 for large requests (fewer atomic adds on
// the arena counter), 1 for small ones (enough workgroups to fill the GPU).
constexpr int kLookupItemsLarge = 4;
constexpr uint64_t kLookupLargeKeys = 1u << 20;

// FIXED: find or create the row of every key. Push and pull both create
// (pull of an absent key inserts a zero value, kv_app.h:457).
// A round handles kBlock*kLookupItems keys, kLookupItems consecutive ones per thread:
// every thread claims slots for its keys, then the workgroup takes the rows of all
// created keys from the arena with ONE atomic add and a workgroup-wide scan hands them
// out in request order, so rows of neighbouring keys are neighbours in the arena.
// FIXED: request `tag` repeats a key. Reported by the next wait; the request's row kernels
// change no stored value.
__device__ __forceinline__ void refuse_fixed(DevState* st, const ReqTag& tag) {
  atomicOr(&st->error, kDevErrDuplicate);
  st->bad_epoch = tag.epoch;
  st->refused_epoch = tag.epoch;
}

template <int kLookupItems>
__global__ __launch_bounds__(kBlock) void k_lookup_fixed(ReqBatch b) {
  const TableReq& d = b.t[blockIdx.y];
  const unsigned nblk = d.nblk;
  if (blockIdx.x >= nblk) return;
  Slot* __restrict__ slots = d.slots;
  const uint64_t mask = d.mask;
  DevState* st = d.st;
  const uint64_t* __restrict__ keys = d.keys;
  const uint64_t n = d.n;
  uint64_t* __restrict__ ref = d.ref;
  uint64_t* __restrict__ cache_keys = d.cache_keys;
  const ReqTag tag = d.tag;
  Snapshot* snap = d.snap;
  const uint64_t snap_seq = d.snap_seq;
  if (cache_same(st, tag)) {  // the references of the cached request are this request's
    if (snap && blockIdx.x == 0 && threadIdx.x < 64) publish_snapshot(st, snap, snap_seq);
    return;
  }
  if (tag.replay) return;
  if (blockIdx.x == 0 && threadIdx.x == 0) st->cache_epoch = cache_keys ? tag.epoch : 0ull;
  __shared__ unsigned long long red[kBlock / 64];
  __shared__ unsigned cred[kBlock / 64];
  __shared__ unsigned long long s_first;
  __shared__ unsigned s_last;
  unsigned created = 0;
  constexpr uint64_t kRound = (uint64_t)kBlock * kLookupItems;
  for (uint64_t base = (uint64_t)blockIdx.x * kRound; base < n; base += (uint64_t)nblk * kRound) {
    uint64_t* p[kLookupItems];
    uint64_t seen[kLookupItems];
    bool is_new[kLookupItems];
    unsigned mine = 0;
#pragma unroll
    for (int j = 0; j < kLookupItems; ++j) {
      const uint64_t i = base + (uint64_t)threadIdx.x * kLookupItems + j;
      p[j] = nullptr;
      is_new[j] = false;
      seen[j] = 0;
      if (i < n) {
        const uint64_t key = keys[i];
        if (cache_keys) cache_keys[i] = key;
        // keys are sorted and must be unique (kv_app.h:17): a key that equals its left neighbour
        // refuses the request, whether the key is new or has been in the table for long
        if (i > 0 && keys[i - 1] == key) {
          refuse_fixed(st, tag);
        } else {
          p[j] = find_or_insert(slots, mask, st, key, is_new[j], seen[j]);
        }
      }
      if (p[j] && !is_new[j] && seen[j] == kPayloadUnset) {
        // (unsorted request) another lane of this request is creating the very same key
        refuse_fixed(st, tag);
        p[j] = nullptr;
      }
      mine += (p[j] && is_new[j]) ? 1u : 0u;
    }
    unsigned long long total;
    unsigned long long at = block_excl_scan_u64(mine, red, total);
    if (threadIdx.x == 0 && total) s_first = atomicAdd(&st->arena_top, total);
    __syncthreads();
    at += total ? s_first : 0ull;
#pragma unroll
    for (int j = 0; j < kLookupItems; ++j) {
      const uint64_t i = base + (uint64_t)threadIdx.x * kLookupItems + j;
      if (i >= n) continue;
      if (!p[j]) {
        ref[i] = kRefAbsent;
        continue;
      }
      uint64_t row = seen[j];
      if (is_new[j]) {
        row = at++;
        *p[j] = row;
      }
      ref[i] = row | (is_new[j] ? kRefNew : 0ull);
    }
    created += mine;
    __syncthreads();  // s_first and red are reused by the next round
  }
  block_count_add(st, created, cred);
  publish_after_lookup(st, snap, snap_seq, nblk, &s_last);
}

// VARLEN push, first kernel: one pass over the request's keys and lens that
//   - compares them with the cached request (when the host found the cache usable),
//   - takes pass 1 of the lens scan (per-workgroup totals, flags),
// and whose last workgroup decides whether the request repeats the cached one and scans the
// totals. Always launched for a push, so the decision and the scan cost no launch of their
// own.
template <int kItems>
__global__ __launch_bounds__(kBlock) void k_var_push_begin(ReqBatch b) {
  const TableReq& d = b.t[blockIdx.y];
  const unsigned nblk = d.nblk;
  if (blockIdx.x >= nblk) return;
  const uint64_t* __restrict__ keys = d.keys;
  const int32_t* __restrict__ lens = d.lens;
  const uint64_t n = d.n;
  const uint64_t* __restrict__ cache_keys = d.cache_keys;
  const int32_t* __restrict__ cache_lens = d.cache_lens;
  unsigned long long* __restrict__ part = d.part;
  DevState* st = d.st;
  constexpr unsigned max_len = PSKV_MAX_VARLEN_ROW;
  const ReqTag tag = d.tag;
  __shared__ unsigned long long red[kBlock / 64];
  __shared__ unsigned fred[kBlock / 64];
  __shared__ unsigned long long carry_s;
  __shared__ unsigned s_last;
  const uint64_t base = ((uint64_t)blockIdx.x * kBlock + threadIdx.x) * kItems;
  // all loads first, then the arithmetic
  int32_t l[kItems], cl[kItems];
  uint64_t k[kItems], ck[kItems];
#pragma unroll
  for (int j = 0; j < kItems; ++j) {
    const bool in = base + j < n;
    l[j] = in ? lens[base + j] : 0;
    k[j] = in ? keys[base + j] : 0;
    ck[j] = k[j];
    cl[j] = l[j];
    if (in && tag.try_cache) {
      ck[j] = cache_keys[base + j];
      cl[j] = cache_lens[base + j];
    }
  }
  // the key in front of this thread's first one (its neighbour has asked for that line already)
  const uint64_t left = (base > 0 && base < n) ? keys[base - 1] : 0;
  unsigned long long s = 0;
  unsigned flags = 0;
#pragma unroll
  for (int j = 0; j < kItems; ++j) {
    s += (unsigned long long)(long long)l[j];
    flags |= (unsigned)l[j] & kReqMisaligned;
    flags |= (l[j] < 0 || (unsigned)l[j] > max_len) ? kReqBadLen : 0u;
    flags |= (k[j] != ck[j] || l[j] != cl[j]) ? kReqDiffer : 0u;
    // keys are sorted and must be unique (kv_app.h:17): a key that equals its left neighbour
    // refuses the request before anything of it is applied
    const bool has_left = base + j < n && base + j > 0;
    flags |= (has_left && k[j] == (j ? k[j - 1] : left)) ? kReqDuplicate : 0u;
  }
  if (!scan_pass1_block(s, flags, part, st, nblk, red, fred, &s_last)) return;
  flags = scan_pass1_last(part, st, nblk, tag.epoch, red, &carry_s);
  if (threadIdx.x == 0) decide_same(st, tag, (flags & kReqDiffer) != 0u, d.outcome);
}

// VARLEN push, second kernel: pass 2 of the lens scan (request-side offsets and the tile
// table) and, for the same keys, find-or-create: a created row gets ceil(len/4) 16-byte
// units of the arena, so every row starts 16-byte aligned; a present row must have the
// pushed length. A workgroup handles kBlock*kItems consecutive keys: every thread claims
// slots for its keys, then the workgroup takes the rows of all created keys from the arena
// with ONE atomic add and a workgroup-wide scan hands them out in request order, so rows of
// neighbouring keys are neighbours in the arena.
constexpr unsigned long long kArenaPadUnits = 8;  // 128 bytes in 16-byte allocation units

template <int kItems>
__global__ __launch_bounds__(kBlock) void k_var_push_lookup(ReqBatch b) {
  const TableReq& d = b.t[blockIdx.y];
  const unsigned nblk = d.nblk;
  if (blockIdx.x >= nblk) return;
  Slot* __restrict__ slots = d.slots;
  const uint64_t mask = d.mask;
  DevState* st = d.st;
  const uint64_t* __restrict__ keys = d.keys;
  const int32_t* __restrict__ lens = d.lens;
  const uint64_t n = d.n, nvals = d.nvals;
  const unsigned long long* __restrict__ part = d.part;
  uint64_t* __restrict__ off = d.off;
  uint32_t* __restrict__ tile_key = d.tile_key;
  const uint64_t ntiles = d.ntiles;
  constexpr uint64_t tile = PSKV_TILE_VAR;
  uint64_t* __restrict__ ref = d.ref;
  uint64_t* __restrict__ cache_keys = d.cache_keys;
  int32_t* __restrict__ cache_lens = d.cache_lens;
  const ReqTag tag = d.tag;
  Snapshot* snap = d.snap;
  const uint64_t snap_seq = d.snap_seq;
  if (cache_same(st, tag)) {  // offsets, tile table and references of the cached request hold
    if (snap && blockIdx.x == 0 && threadIdx.x < 64) publish_snapshot(st, snap, snap_seq);
    return;
  }
  if (tag.replay) return;
  // the request is refused as a whole when its lens are invalid or do not add up to vals.size(),
  // or when it repeats a key
  // (a refused request creates nothing, so the counter record the host may be waiting for holds
  // the counters as they are)
  if (st->req_error & (kDevErrBadLen | kDevErrSizeMismatch | kDevErrDuplicate)) {
    if (snap && blockIdx.x == 0 && threadIdx.x < 64) publish_snapshot(st, snap, snap_seq);
    return;
  }
  if (st->scan_total != nvals) {
    if (blockIdx.x == 0 && threadIdx.x == 0) raise_error(st, kDevErrSizeMismatch, tag.epoch);
    if (snap && blockIdx.x == 0 && threadIdx.x < 64) publish_snapshot(st, snap, snap_seq);
    return;
  }
  __shared__ unsigned long long wsum[kBlock / 64];
  __shared__ unsigned long long red[kBlock / 64];
  __shared__ unsigned cred[kBlock / 64];
  __shared__ unsigned long long s_first;
  __shared__ unsigned s_last;
  const uint64_t base = ((uint64_t)blockIdx.x * kBlock + threadIdx.x) * kItems;
  unsigned long long len[kItems];
#pragma unroll
  for (int j = 0; j < kItems; ++j) len[j] = base + j < n ? (unsigned long long)(uint32_t)lens[base + j] : 0ull;
  scan_pass2_offsets<kItems>(len, base, n, part[blockIdx.x], off, tile_key, ntiles, tile, wsum);

  uint64_t* p[kItems];
  uint64_t seen[kItems];
  bool is_new[kItems];
  unsigned long long units = 0;
  unsigned mine = 0;
#pragma unroll
  for (int j = 0; j < kItems; ++j) {
    const uint64_t i = base + j;
    p[j] = nullptr;
    is_new[j] = false;
    seen[j] = 0;
    if (i < n) {
      const uint64_t key = keys[i];
      cache_keys[i] = key;
      cache_lens[i] = (int32_t)len[j];
      p[j] = find_or_insert(slots, mask, st, key, is_new[j], seen[j]);
      if (p[j] && !is_new[j] && seen[j] == kPayloadUnset) {
        atomicOr(&st->error, kDevErrDuplicate);  // the same key twice in this request
        st->bad_epoch = tag.epoch;
        p[j] = nullptr;
      }
    }
    if (p[j] && is_new[j]) {
      units += (len[j] + 3) >> 2;
      ++mine;
    }
  }
  unsigned long long total;
  unsigned long long at = block_excl_scan_u64(units, red, total);
  if (threadIdx.x == 0 && total) {
    // kArenaPadUnits - 1 units of slack let the workgroup's rows start at an arena address that
    // is congruent, modulo 128 bytes, to the request-side offset of the workgroup's first key.
    // When all its keys are new (a first push) the rows then mirror the request 128-byte line
    // for 128-byte line, and the row kernels' arena accesses are as aligned as their
    // request-side ones (misaligned ones cost about 5 % of their bandwidth).
    const unsigned long long first = atomicAdd(&st->arena_top, total + (kArenaPadUnits - 1));
    const unsigned long long want = (part[blockIdx.x] >> 2) & (kArenaPadUnits - 1);
    s_first = first + ((want - first) & (kArenaPadUnits - 1));
  }
  __syncthreads();
  at += total ? s_first : 0ull;
#pragma unroll
  for (int j = 0; j < kItems; ++j) {
    const uint64_t i = base + j;
    if (i >= n) continue;
    if (!p[j]) {
      ref[i] = kRefAbsent;
      continue;
    }
    uint64_t payload = seen[j];
    if (is_new[j]) {
      payload = ((uint64_t)at << kLenBits) | len[j];
      at += (len[j] + 3) >> 2;
      *p[j] = payload;
    } else if ((payload & kLenMask) != len[j]) {
      raise_error(st, kDevErrLenChanged, tag.epoch);
    }
    ref[i] = payload | (is_new[j] ? kRefNew : 0ull);
  }
  block_count_add(st, mine, cred);
  publish_after_lookup(st, snap, snap_seq, nblk, &s_last);
}

// VARLEN pull, first kernel: the stored length of every key (an absent key answers length 0
// and is not created) together with pass 1 of the scan over those lengths. With the keys of
// the cached push the answer is known without a single probe: every key is present with the
// cached length, and the offsets of that push are the offsets of this response.
template <int kItems>
__global__ __launch_bounds__(kBlock) void k_var_pull_lookup(ReqBatch b) {
  const TableReq& d = b.t[blockIdx.y];
  const unsigned nblk = d.nblk;
  if (blockIdx.x >= nblk) return;
  const Slot* __restrict__ slots = d.slots;
  const uint64_t mask = d.mask;
  DevState* st = d.st;
  const uint64_t* __restrict__ keys = d.keys;
  const uint64_t n = d.n;
  uint64_t* __restrict__ ref = d.ref;
  int32_t* __restrict__ out_lens = d.out_lens;
  const int32_t* __restrict__ cache_lens = d.cache_lens;
  unsigned long long* __restrict__ part = d.part;
  const ReqTag tag = d.tag;
  __shared__ unsigned long long red[kBlock / 64];
  __shared__ unsigned fred[kBlock / 64];
  __shared__ unsigned long long carry_s;
  __shared__ unsigned s_last;
  const uint64_t base = ((uint64_t)blockIdx.x * kBlock + threadIdx.x) * kItems;
  if (cache_same(st, tag)) {
#pragma unroll
    for (int j = 0; j < kItems; ++j)
      if (base + j < n) out_lens[base + j] = cache_lens[base + j];
    return;
  }
  if (tag.replay) return;
  // this pull rewrites the references and offsets in the workspace: the cached push is gone
  if (blockIdx.x == 0 && threadIdx.x == 0) st->bad_epoch = st->cache_epoch;
  unsigned long long s = 0;
  unsigned bits = 0;
#pragma unroll
  for (int j = 0; j < kItems; ++j) {
    const uint64_t i = base + j;
    if (i < n) {
      uint64_t payload;
      const bool hit = find_only(slots, mask, st, keys[i], payload);
      const uint32_t l = hit ? (uint32_t)(payload & kLenMask) : 0u;
      ref[i] = hit ? payload : kRefAbsent;
      out_lens[i] = (int32_t)l;
      s += l;
      bits |= l & 3u;
    }
  }
  if (!scan_pass1_block(s, bits, part, st, nblk, red, fred, &s_last)) return;
  scan_pass1_last(part, st, nblk, tag.epoch, red, &carry_s);
}

// VARLEN pull, second kernel: pass 2 of the scan over the answered lengths: the request-side
// offsets of the response and its tile table. `ntiles_cap` is the room in the table; the
// tiles in use follow from the scanned total.
template <int kItems>
__global__ __launch_bounds__(kBlock) void k_var_offsets(ReqBatch b) {
  const TableReq& d = b.t[blockIdx.y];
  if (blockIdx.x >= d.nblk) return;
  const int32_t* __restrict__ lens = d.out_lens;  // the lengths the lookup kernel answered
  const uint64_t n = d.n;
  const unsigned long long* __restrict__ part = d.part;
  uint64_t* __restrict__ off = d.off;
  uint32_t* __restrict__ tile_key = d.tile_key;
  const uint64_t ntiles_cap = d.ntiles;
  constexpr uint64_t tile = PSKV_TILE_VAR;
  const DevState* st = d.st;
  const ReqTag tag = d.tag;
  if (cache_same(st, tag) || tag.replay) return;  // offsets and tile table of the cached request hold
  __shared__ unsigned long long wsum[kBlock / 64];
  uint64_t ntiles = (st->scan_total + tile - 1) / tile;
  if (ntiles > ntiles_cap) ntiles = ntiles_cap;
  const uint64_t base = ((uint64_t)blockIdx.x * kBlock + threadIdx.x) * kItems;
  unsigned long long len[kItems];
#pragma unroll
  for (int j = 0; j < kItems; ++j) len[j] = base + j < n ? (unsigned long long)(uint32_t)lens[base + j] : 0ull;
  scan_pass2_offsets<kItems>(len, base, n, part[blockIdx.x], off, tile_key, ntiles, tile, wsum);
}

// ---------------------------------------------------------------------------------
// Row modes, step 2: stream the values.
// A workgroup owns one tile of consecutive floats of the request-side
// buffer, whatever rows they belong to, so the load is balanced for any mix of row
// lengths and the request side is read or written fully coalesced with 128-bit
// accesses. FIXED locates the row of an element by division; VARLEN stages the
// offsets and row references of the keys that overlap the tile in LDS and locates
// rows by binary search there.
// ---------------------------------------------------------------------------------
struct RowsParams {
  float* req;                // push: request values (read); pull: response values (written)
  float* arena;              // row storage
  const uint64_t* ref;       // n row references from the lookup kernel
  const uint64_t* off;       // VARLEN: n+1 request-side row offsets in floats
  const uint32_t* tile_key;  // VARLEN: ntiles+1 entries
  TileNote* tile_aff;        // VARLEN: one note per tile
  DevState* st;
  uint64_t n;
  uint64_t total;         // floats in req
  uint64_t k;             // FIXED: floats per row
  uint32_t force_scalar;  // request buffer or k not 16-byte friendly
  uint32_t ignore_new;    // pull half of a push+pull: rows created by the push half hold data
  uint32_t total_on_device;  // VARLEN pull without a host round trip: the floats to move are
                             // DevState::scan_total and `total` is the room in req
  uint32_t blk;              // the workgroup's number among those that cover the request
  ReqTag tag;
};

constexpr int kOpAcc = 0;
constexpr int kOpGather = 1;

// VEC floats moved by one lane per access. STREAM selects non-temporal accesses: a
// request far larger than the caches is read and written once per launch, and telling
// the memory system so is worth 10-15 % of bandwidth on this GPU.
template <int VEC>
struct VecT;
template <>
struct VecT<4> {
  using type = f32x4;
  __device__ static f32x4 zero() { return (f32x4)(0.f); }
};
template <>
struct VecT<1> {
  using type = float;
  __device__ static float zero() { return 0.f; }
};
template <bool STREAM, typename V>
__device__ __forceinline__ V vload(const V* p) {
  return STREAM ? __builtin_nontemporal_load(p) : *p;
}
template <bool STREAM, typename V>
__device__ __forceinline__ void vstore(V v, V* p) {
  if (STREAM) __builtin_nontemporal_store(v, p); else *p = v;
}

// FIXED rows: a workgroup owns TILE consecutive request-side floats; the row of an element
// follows from a division (one compare when a row is at least a tile long).
template <int OP, int VEC, bool STREAM, unsigned TILE>
__device__ __forceinline__ void rows_tile_fixed(const RowsParams& p, uint64_t total) {
  // a refused push (it repeats a key) changes no stored value; rows it created stay, as zero rows
  const bool rejected = OP == kOpAcc && p.st->refused_epoch == p.tag.epoch;
  using V = typename VecT<VEC>::type;
  constexpr int kIter = TILE / (VEC * kBlock);      // elements per thread
  constexpr int kGroup = kIter < 4 ? kIter : 4;     // loads issued back to back
  static_assert(kIter >= 1 && kIter % kGroup == 0, "tile does not divide over the workgroup");
  const uint64_t f0 = (uint64_t)p.blk * TILE;
  if (f0 >= total) return;
  const uint32_t tile_floats = (uint32_t)((total - f0 < (uint64_t)TILE) ? (total - f0) : (uint64_t)TILE);
  const uint32_t nelem = tile_floats / VEC;

  // The request-side loads depend on nothing but the tile index: issue them first so that
  // they are in flight while the row references are fetched.
  V x[kIter];
  if (OP == kOpAcc) {
#pragma unroll
    for (int i = 0; i < kIter; ++i) {
      const uint32_t le = (uint32_t)i * kBlock + threadIdx.x;
      x[i] = VecT<VEC>::zero();
      if (le < nelem) x[i] = vload<STREAM>(reinterpret_cast<const V*>(p.req + f0 + le * VEC));
    }
  }
  const uint64_t j0 = f0 / p.k;           // row of the tile's first float
  const uint64_t rem0 = f0 - j0 * p.k;    // and its offset in that row

#pragma unroll
  for (int g = 0; g < kIter; g += kGroup) {
    V y[kGroup];
    V* dst[kGroup];
    uint32_t lf[kGroup];
    bool live[kGroup], fresh[kGroup];
#pragma unroll
    for (int u = 0; u < kGroup; ++u) {
      const uint32_t le = (uint32_t)(g + u) * kBlock + threadIdx.x;
      live[u] = le < nelem;
      lf[u] = le * VEC;
      dst[u] = nullptr;
      fresh[u] = false;
      if (!live[u]) continue;
      const uint64_t xoff = rem0 + lf[u];
      uint64_t q, within;
      if (p.k >= (uint64_t)TILE) {
        q = xoff >= p.k ? 1u : 0u;
        within = q ? xoff - p.k : xoff;
      } else {
        const uint32_t q32 = (uint32_t)xoff / (uint32_t)p.k;
        q = q32;
        within = (uint32_t)xoff - q32 * (uint32_t)p.k;
      }
      const uint64_t r = p.ref[j0 + q];
      dst[u] = reinterpret_cast<V*>(p.arena + (r & ~kRefNew) * p.k + within);
      if (r == kRefAbsent) {  // a key the lookup refused (duplicate in the request, full table)
        live[u] = false;
        continue;
      }
      fresh[u] = (r & kRefNew) != 0 && !p.ignore_new;
    }
    // all stored-row loads of the group before the first add
#pragma unroll
    for (int u = 0; u < kGroup; ++u) {
      y[u] = VecT<VEC>::zero();
      if (live[u] && !fresh[u]) y[u] = vload<STREAM>(dst[u]);
    }
#pragma unroll
    for (int u = 0; u < kGroup; ++u) {
      if (!live[u]) continue;
      if (OP == kOpAcc) {
        if (rejected) {
          if (fresh[u]) vstore<STREAM>(VecT<VEC>::zero(), dst[u]);
        } else {
          // a created row is a zero row first (0.0f + v), kv_app.h:454
          vstore<STREAM>(y[u] + x[g + u], dst[u]);
        }
      } else {
        vstore<STREAM>(y[u], reinterpret_cast<V*>(p.req + f0 + lf[u]));
        if (fresh[u]) vstore<STREAM>(VecT<VEC>::zero(), dst[u]);  // pull created the row: zeros
      }
    }
  }
}

// VARLEN rows: a WAVEFRONT owns WTILE consecutive request-side floats. The tile table names
// the first key that overlaps them; the wavefront stages the offsets and row references of
// the keys that overlap its tile in its own piece of LDS (no workgroup barrier: the four
// wavefronts of a workgroup never wait for each other) and finds the row of each element by
// binary search there. Tiles that overlap more than kWaveSpan keys (rows of a float or two)
// search the global arrays instead.
constexpr unsigned kWaveSpan = 128;

// What a wavefront can ask for knowing nothing but its tile index: the tile's shortcut note (read
// even when it turns out not to be needed, so that it is not a second round trip after the
// decision) and the request-side values. `bound` is what the host knows of the request's
// length; the data may be shorter.
template <int OP, int VEC, bool STREAM, unsigned WTILE>
__device__ __forceinline__ void rows_wave_ask(const RowsParams& p, uint64_t bound,
                                              typename VecT<VEC>::type* x, TileNote& aff) {
  using V = typename VecT<VEC>::type;
  constexpr int kIter = WTILE / (VEC * 64);
  const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint64_t wt = (uint64_t)p.blk * (kBlock / 64) + wave;
  const uint64_t f0 = wt * WTILE;
  const uint64_t left = bound > f0 ? bound - f0 : 0;  // 0: the tile lies past the data
  const uint32_t nelem = (uint32_t)(left < (uint64_t)WTILE ? left : (uint64_t)WTILE) / VEC;
  aff.first = kTileNotAffine;
  aff.second = 0;
  if (VEC == 4 && left) {
    const u64x2 w = *reinterpret_cast<const u64x2*>(&p.tile_aff[wt]);  // one 128-bit load
    aff.first = w.x;
    aff.second = w.y;
  }
  if (OP == kOpAcc) {
#pragma unroll
    for (int i = 0; i < kIter; ++i) {
      const uint32_t le = (uint32_t)i * 64 + lane;
      x[i] = VecT<VEC>::zero();
      if (le < nelem) x[i] = vload<STREAM>(reinterpret_cast<const V*>(p.req + f0 + le * VEC));
    }
  }
}

// Shortcut of a request that repeats the cached one: if the rows of this tile lie in the arena
// as one or two unbroken pieces (two: the tile straddles the rows of two workgroups of the
// lookup that created them), the note the row kernel of the cached request left maps every
// float with an offset and neither the row table nor a search is needed. Returns false when the
// tile has to take the general way. Wavefront-uniform.
template <int OP, bool STREAM, unsigned WTILE>
__device__ __forceinline__ bool rows_wave_affine(const RowsParams& p, uint64_t total,
                                                 const f32x4* x, const TileNote& aff) {
  using V = f32x4;
  constexpr int VEC = 4;
  constexpr int kIter = WTILE / (VEC * 64);
  static_assert(WTILE < (1u << kTileSplitBits), "the split index does not fit the note");
  if (aff.first == kTileNotAffine) return false;
  const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint64_t wt = (uint64_t)p.blk * (kBlock / 64) + wave;
  const uint64_t f0 = wt * WTILE;
  if (f0 >= total) return true;
  const uint32_t nelem = (uint32_t)((total - f0 < (uint64_t)WTILE) ? (total - f0) : (uint64_t)WTILE) / VEC;
  // rows start on multiples of four floats here, so no 128-bit element straddles the split
  const uint32_t split = aff.second ? (uint32_t)(aff.second & ((1u << kTileSplitBits) - 1)) : ~0u;
  const int64_t first = (int64_t)aff.first;
  const int64_t second = (int64_t)(aff.second >> kTileSplitBits) - kTileNoteBias;  // may be negative
  V y[kIter];
  V* dst[kIter];
#pragma unroll
  for (int i = 0; i < kIter; ++i) {
    const uint32_t le = (uint32_t)i * 64 + lane;
    dst[i] = reinterpret_cast<V*>(p.arena + ((le * VEC >= split ? second : first) + (int64_t)(le * VEC)));
    y[i] = VecT<VEC>::zero();
    if (le < nelem) y[i] = vload<STREAM>(dst[i]);
  }
#pragma unroll
  for (int i = 0; i < kIter; ++i) {
    const uint32_t le = (uint32_t)i * 64 + lane;
    if (le >= nelem) continue;
    if (OP == kOpAcc) {
      vstore<STREAM>(y[i] + x[i], dst[i]);
    } else {
      vstore<STREAM>(y[i], reinterpret_cast<V*>(p.req + f0 + le * VEC));
    }
  }
  return true;
}

// `x` comes from rows_wave_ask; x[i] is used only below `total`.
template <int OP, int VEC, bool STREAM, unsigned WTILE>
__device__ __forceinline__ void rows_wave_varlen(const RowsParams& p, uint64_t total,
                                                 int32_t* s_off_all, uint64_t* s_ref_all,
                                                 bool rejected, bool same,
                                                 const typename VecT<VEC>::type* x) {
  using V = typename VecT<VEC>::type;
  constexpr int kIter = WTILE / (VEC * 64);  // elements per lane
  static_assert(kIter >= 1 && kIter <= 8, "wave tile out of range");
  const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint64_t wt = (uint64_t)p.blk * (kBlock / 64) + wave;
  const uint64_t f0 = wt * WTILE;
  if (f0 >= total) return;  // the whole wavefront leaves; nothing below synchronises workgroups
  const uint32_t tile_floats = (uint32_t)((total - f0 < (uint64_t)WTILE) ? (total - f0) : (uint64_t)WTILE);
  const uint32_t nelem = tile_floats / VEC;

  const uint64_t j_lo = p.tile_key[wt];
  const uint32_t span = (uint32_t)((uint64_t)p.tile_key[wt + 1] - j_lo + 1);
  const bool staged = span <= kWaveSpan;
  int32_t* s_off = s_off_all + wave * (kWaveSpan + 1);
  uint64_t* s_ref = s_ref_all + wave * kWaveSpan;
  if (staged) {
    for (uint32_t s = lane; s <= span; s += 64) {
      s_off[s] = (int32_t)(int64_t)(p.off[j_lo + s] - f0);
      if (s < span) s_ref[s] = p.ref[j_lo + s];
    }
    // the wavefront's own LDS writes, visible to all of its lanes before the reads below
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  if (!same) {
    // Leave a note for requests that repeat this one. Every row with floats in the tile has a
    // distance between its place in the arena and its place in the request; the tile is one
    // piece when all distances are equal (the rows lie back to back, in request order, without
    // padding between them) and two pieces when they change once.
    TileNote note = {kTileNotAffine, 0};
    if (VEC == 4 && staged) {
      bool absent = false;
      int64_t d[(kWaveSpan + 63) / 64];
      bool has[(kWaveSpan + 63) / 64];
#pragma unroll
      for (uint32_t it = 0; it < (kWaveSpan + 63) / 64; ++it) {
        const uint32_t s = it * 64 + lane;
        has[it] = s < span && s_off[s + 1] > s_off[s] && s_off[s] < (int32_t)tile_floats;
        d[it] = 0;
        if (has[it]) {
          const uint64_t r = s_ref[s];
          absent |= r == kRefAbsent;
          d[it] = (int64_t)(((r & ~kRefNew) >> kLenBits) << 2) - (int64_t)s_off[s];
        }
      }
      // the first row with floats, its distance, and the first row whose distance differs
      uint32_t s0 = ~0u, s1 = ~0u;
#pragma unroll
      for (uint32_t it = 0; it < (kWaveSpan + 63) / 64; ++it) {
        const uint64_t m = __ballot(has[it]);
        if (s0 == ~0u && m) s0 = it * 64 + (uint32_t)__builtin_ctzll(m);
      }
      if (s0 != ~0u && __ballot(absent) == 0ull) {
        const uint64_t r0 = s_ref[s0];
        const int64_t d0 = (int64_t)(((r0 & ~kRefNew) >> kLenBits) << 2) - (int64_t)s_off[s0];
#pragma unroll
        for (uint32_t it = 0; it < (kWaveSpan + 63) / 64; ++it) {
          const uint64_t m = __ballot(has[it] && d[it] != d0);
          if (s1 == ~0u && m) s1 = it * 64 + (uint32_t)__builtin_ctzll(m);
        }
        if (s1 == ~0u) {
          note.first = (uint64_t)d0;
        } else {
          const uint64_t r1 = s_ref[s1];
          const int32_t at = s_off[s1];  // > 0: row s0 comes first and has floats in the tile
          const int64_t d1 = (int64_t)(((r1 & ~kRefNew) >> kLenBits) << 2) - (int64_t)at;
          bool other = false;
#pragma unroll
          for (uint32_t it = 0; it < (kWaveSpan + 63) / 64; ++it)
            other |= has[it] && it * 64 + lane > s1 && d[it] != d1;
          if (__ballot(other) == 0ull && at > 0) {
            note.first = (uint64_t)d0;
            note.second = ((uint64_t)(d1 + kTileNoteBias) << kTileSplitBits) | (uint64_t)(uint32_t)at;
          }
        }
      }
    }
    if (lane == 0) p.tile_aff[wt] = note;
  }

  V y[kIter];
  V* dst[kIter];
  bool live[kIter], fresh[kIter];
#pragma unroll
  for (int i = 0; i < kIter; ++i) {
    const uint32_t le = (uint32_t)i * 64 + lane;
    const uint32_t lf = le * VEC;
    live[i] = le < nelem;
    dst[i] = nullptr;
    fresh[i] = false;
    if (!live[i]) continue;
    uint64_t r, within;
    if (staged) {
      // last key whose first float is at or before lf (zero-length rows repeat an offset)
      uint32_t lo = 0, hi = span;
      while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (s_off[mid] <= (int32_t)lf) lo = mid + 1; else hi = mid;
      }
      r = s_ref[lo - 1];
      within = (uint64_t)((int32_t)lf - s_off[lo - 1]);
    } else {
      const uint64_t f = f0 + lf;
      uint64_t lo = j_lo, hi = j_lo + span;
      while (lo < hi) {
        const uint64_t mid = (lo + hi) >> 1;
        if (p.off[mid] <= f) lo = mid + 1; else hi = mid;
      }
      r = p.ref[lo - 1];
      within = f - p.off[lo - 1];
    }
    dst[i] = reinterpret_cast<V*>(p.arena + (((r & ~kRefNew) >> kLenBits) << 2) + within);
    if (r == kRefAbsent) {  // a key the lookup refused (duplicate in the request, full table)
      live[i] = false;
      continue;
    }
    fresh[i] = (r & kRefNew) != 0 && !p.ignore_new;
  }
#pragma unroll
  for (int i = 0; i < kIter; ++i) {
    y[i] = VecT<VEC>::zero();
    if (live[i] && !fresh[i]) y[i] = vload<STREAM>(dst[i]);
  }
#pragma unroll
  for (int i = 0; i < kIter; ++i) {
    if (!live[i]) continue;
    const uint32_t lf = ((uint32_t)i * 64 + lane) * VEC;
    if (OP == kOpAcc) {
      if (rejected) {
        // a refused push changes no stored value; rows it created stay, as zero rows
        if (fresh[i]) vstore<STREAM>(VecT<VEC>::zero(), dst[i]);
      } else {
        vstore<STREAM>(y[i] + x[i], dst[i]);  // a created row is a zero row first (0.0f + v)
      }
    } else {
      vstore<STREAM>(y[i], reinterpret_cast<V*>(p.req + f0 + lf));
    }
  }
}

// Request-side floats per workgroup (fixed rows) and per wavefront (var-len rows). One
// 128-bit access per lane and many small workgroups stream fastest on this GPU (6.5 TB/s for
// `row += in` against 5.5 TB/s with four accesses per lane).
constexpr unsigned kTileFixed = 1024;
constexpr unsigned kTileVar = PSKV_TILE_VAR;        // per wavefront; the tile table's granularity
constexpr unsigned kRowsVarPerBlock = kTileVar * (kBlock / 64);

template <int OP, bool VARLEN, bool STREAM>
__global__ __launch_bounds__(kBlock) void k_rows(ReqBatch b) {
  const TableReq& d = b.t[blockIdx.y];
  // the grid is sized for the largest table of the launch: workgroups (VARLEN: wavefronts) past
  // this table's floats leave before they touch anything
  if ((((uint64_t)blockIdx.x + d.tile_base) * (kBlock / 64) + (VARLEN ? (threadIdx.x >> 6) : 0u)) *
          (VARLEN ? kTileVar : kTileFixed / (kBlock / 64)) >= d.total)
    return;
  RowsParams p;
  p.req = d.req;
  p.arena = d.arena;
  p.ref = d.ref;
  p.off = d.off;
  p.tile_key = d.tile_key;
  p.tile_aff = d.tile_aff;
  p.st = d.st;
  p.n = d.n;
  p.total = d.total;
  p.k = d.k;
  p.force_scalar = d.force_scalar;
  p.ignore_new = d.ignore_new;
  p.total_on_device = d.total_on_device;
  p.blk = blockIdx.x + d.tile_base;
  p.tag = d.tag;
  __shared__ int32_t s_off[VARLEN ? (kWaveSpan + 1) * (kBlock / 64) : 1];
  __shared__ uint64_t s_ref[VARLEN ? kWaveSpan * (kBlock / 64) : 1];
  bool rejected = false;
  bool scalar = p.force_scalar != 0;
  uint64_t total = p.total;
  // What the device knows about the request: one load, one wait per wavefront.
  const ReqFacts facts = load_req_facts(p.st);
  if (VARLEN) {
    // every argument the common path uses, asked for at once (the compiler otherwise fetches them
    // group by group where they are first used, one wait each)
    asm volatile("" ::"s"(p.req), "s"(p.arena), "s"(p.tile_aff), "s"(p.total),
                 "s"(p.force_scalar), "s"(p.total_on_device), "s"(p.tag.epoch));
  }
  if (VARLEN) {
    // the grid covers the room in the caller's buffer, which may be more than the data
    const uint64_t f0 = ((uint64_t)p.blk * (kBlock / 64) + (threadIdx.x >> 6)) * kTileVar;
    if (f0 >= p.total) return;
    // the loads that need no facts are on their way before the facts are looked at
    f32x4 x4[kTileVar / 256];
    TileNote aff = {kTileNotAffine, 0};
    if (!scalar) rows_wave_ask<OP, 4, STREAM, kTileVar>(p, p.total, x4, aff);
    // a request served from the cached references creates nothing and cannot have been refused
    const bool same = facts.same_epoch == p.tag.epoch;
    if (p.tag.replay && !same) return;
    if (same) p.ignore_new = 1;
    const unsigned err = same ? 0u : facts.req_error;
    if (err & (kDevErrBadLen | kDevErrSizeMismatch | kDevErrDuplicate)) return;
    rejected = (err & kDevErrLenChanged) != 0;
    scalar = scalar || (facts.misaligned != 0);
    if (p.total_on_device) {
      total = facts.scan_total;
      if (total > p.total) {  // the response does not fit the caller's buffer: write nothing
        if (p.blk == 0 && threadIdx.x == 0) atomicOr(&p.st->error, kDevErrNoRoom);
        return;
      }
    }
    if (scalar) {
      float x1[kTileVar / 64];
      TileNote none;
      rows_wave_ask<OP, 1, STREAM, kTileVar>(p, total, x1, none);
      rows_wave_varlen<OP, 1, STREAM, kTileVar>(p, total, s_off, s_ref, rejected, same, x1);
    } else {
      if (same && rows_wave_affine<OP, STREAM, kTileVar>(p, total, x4, aff)) return;
      rows_wave_varlen<OP, 4, STREAM, kTileVar>(p, total, s_off, s_ref, rejected, same, x4);
    }
  } else {
    if (p.tag.replay && facts.same_epoch != p.tag.epoch) return;
    if (facts.same_epoch == p.tag.epoch) p.ignore_new = 1;
    if (scalar) {
      rows_tile_fixed<OP, 1, STREAM, kTileFixed>(p, total);
    } else {
      rows_tile_fixed<OP, 4, STREAM, kTileFixed>(p, total);
    }
  }
}

// ---------------------------------------------------------------------------------
// Maintenance kernels.
// ---------------------------------------------------------------------------------

// Growth, the general way: every live slot of the old array is re-inserted into the new one
// (which starts as all ones); payloads move bit for bit, so stored sums are unchanged.
__global__ __launch_bounds__(kBlock) void k_rehash(const Slot* __restrict__ old_slots,
                                                  uint64_t old_cap, Slot* __restrict__ slots,
                                                  uint64_t mask, DevState* st) {
  const uint64_t stride = (uint64_t)gridDim.x * kBlock;
  for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < old_cap; i += stride) {
    const ulonglong2 s = *reinterpret_cast<const ulonglong2*>(&old_slots[i]);
    if (s.x == kEmptyKey) continue;
    uint64_t h = home_slot(s.x, mask);
    bool placed = false;
    for (uint64_t probes = 0; probes <= mask; ++probes) {
      if (slots[h].key == kEmptyKey) {
        unsigned long long old =
            atomicCAS(reinterpret_cast<unsigned long long*>(&slots[h].key),
                      (unsigned long long)kEmptyKey, (unsigned long long)s.x);
        if (old == kEmptyKey) {
          slots[h].payload = s.y;
          placed = true;
          break;
        }
      }
      h = (h + 1) & mask;
    }
    if (!placed) atomicOr(&st->error, kDevErrFull);
  }
}

// Growth by a small power of two G, as two streaming passes instead of a scatter. A key's home
// slot is the top bits of its hash, so the keys whose homes lie in the old slots [a, a + R) are
// exactly the keys whose new homes lie in [G * a, G * (a + R)): one workgroup builds that
// stretch of the new array in LDS from its R old slots and writes it out whole, empty slots
// included, with coalesced 128-bit stores (the new array needs no fill, and no atomics reach
// memory). What it cannot place there is left for the second pass: keys that sit in its old
// slots but have their home in an earlier stretch (a probe chain that crossed the boundary, or
// wrapped around the end of the array), and keys whose probe chain would leave the LDS stretch.
// The workgroup writes those, packed, over the front of its own old slots (it is the only one
// that reads them) with an empty slot behind the last; k_regrow_rest inserts them the general
// way once every stretch of the new array is in place. At a fill of one half about one key in
// 250 takes the second pass. Payloads move bit for bit.
constexpr int kRegrowOld = kBlock;  // old slots per workgroup, one per thread
constexpr int kRegrowMaxFactor = 8;
__global__ __launch_bounds__(kBlock) void k_regrow(Slot* __restrict__ old_slots, Slot* __restrict__ slots,
                                                  uint64_t old_mask, uint64_t mask, unsigned factor) {
  extern __shared__ unsigned long long regrow_lds[];  // keys of the stretch, then its payloads
  const unsigned T = kRegrowOld * factor;
  unsigned long long* tkey = regrow_lds;
  unsigned long long* tpay = regrow_lds + T;
  __shared__ unsigned long long red[kBlock / 64 + 1];
  const uint64_t a = (uint64_t)blockIdx.x * kRegrowOld;
  const uint64_t A = a * factor;
  const u64x2 s = __builtin_nontemporal_load(reinterpret_cast<const u64x2*>(&old_slots[a + threadIdx.x]));
  for (unsigned j = threadIdx.x; j < T; j += kBlock) {
    tkey[j] = kEmptyKey;
    tpay[j] = kPayloadUnset;
  }
  __syncthreads();
  const bool live = s.x != kEmptyKey;
  bool rest = false;
  if (live) {
    const uint64_t oh = home_slot(s.x, old_mask);
    if (oh >= a && oh <= a + threadIdx.x) {
      unsigned j = (unsigned)(home_slot(s.x, mask) - A);
      rest = true;
      for (; j < T; ++j) {
        if (atomicCAS(&tkey[j], (unsigned long long)kEmptyKey, (unsigned long long)s.x) == kEmptyKey) {
          tpay[j] = s.y;
          rest = false;
          break;
        }
      }
    } else {
      rest = true;  // its home lies in another workgroup's stretch
    }
  }
  unsigned long long total;
  const unsigned long long at = block_excl_scan_u64(rest ? 1ull : 0ull, red, total);  // (two barriers)
  u64x2* out = reinterpret_cast<u64x2*>(slots + A);
  for (unsigned j = threadIdx.x; j < T; j += kBlock) {
    u64x2 v;
    v.x = tkey[j];
    v.y = tpay[j];
    __builtin_nontemporal_store(v, &out[j]);
  }
  // every thread has read its old slot (the barriers of the scan lie in between)
  if (rest) *reinterpret_cast<u64x2*>(&old_slots[a + at]) = s;
  if (threadIdx.x == 0 && total < (unsigned long long)kRegrowOld) old_slots[a + total].key = kEmptyKey;
}

// Second pass of a growth by k_regrow: sixteen lanes per stretch of kRegrowOld old slots read the
// keys the first pass left at its front, up to the first empty slot, and insert them the general way.
constexpr int kRestLanes = 16;
__global__ __launch_bounds__(kBlock) void k_regrow_rest(const Slot* __restrict__ old_slots, uint64_t old_cap,
                                                       Slot* __restrict__ slots, uint64_t mask, DevState* st) {
  const uint64_t stretch = ((uint64_t)blockIdx.x * kBlock + threadIdx.x) / kRestLanes;
  const unsigned l = threadIdx.x % kRestLanes;
  const unsigned group_shift = (threadIdx.x & 63) / kRestLanes * kRestLanes;
  const uint64_t a = stretch * kRegrowOld;
  bool more = a < old_cap;
  for (unsigned c = 0; c < kRegrowOld / kRestLanes; ++c) {
    u64x2 s;
    s.x = kEmptyKey, s.y = 0;
    if (more) s = *reinterpret_cast<const u64x2*>(&old_slots[a + c * kRestLanes + l]);
    // the lanes of a wavefront stay together for the ballot; a group that is done reads nothing
    const unsigned long long ends = __ballot(more && s.x == kEmptyKey);
    const unsigned mine = (unsigned)(ends >> group_shift) & ((1u << kRestLanes) - 1u);
    const unsigned first_end = mine ? (unsigned)__builtin_ctz(mine) : (unsigned)kRestLanes;
    if (more && l < first_end) {
      uint64_t h = home_slot(s.x, mask);
      bool placed = false;
      for (uint64_t probes = 0; probes <= mask; ++probes) {
        if (slots[h].key == kEmptyKey) {
          unsigned long long old = atomicCAS(reinterpret_cast<unsigned long long*>(&slots[h].key),
                                             (unsigned long long)kEmptyKey, (unsigned long long)s.x);
          if (old == kEmptyKey) {
            slots[h].payload = s.y;
            placed = true;
            break;
          }
        }
        h = (h + 1) & mask;
      }
      if (!placed) atomicOr(&st->error, kDevErrFull);
    }
    if (mine) more = false;
    if (!__any(more)) break;
  }
}

// Collects the keys of all live slots (unordered); *counter must start at 0.
__global__ __launch_bounds__(kBlock) void k_collect_keys(const Slot* __restrict__ slots,
                                                        uint64_t cap, uint64_t* __restrict__ out,
                                                        uint64_t out_cap,
                                                        unsigned long long* counter) {
  const uint64_t stride = (uint64_t)gridDim.x * kBlock;
  for (uint64_t base = (uint64_t)blockIdx.x * kBlock; base < cap; base += stride) {
    const uint64_t i = base + threadIdx.x;
    uint64_t key = kEmptyKey;
    if (i < cap) key = slots[i].key;
    const unsigned long long need = key != kEmptyKey ? 1ull : 0ull;
    const unsigned long long inc = wave_incl_scan_u64(need);
    const unsigned long long tot = __shfl(inc, 63);
    unsigned long long first = 0;
    if ((threadIdx.x & 63) == 63 && tot) first = atomicAdd(counter, tot);
    first = __shfl(first, 63);
    const unsigned long long at = first + inc - need;
    if (need && at < out_cap) out[at] = key;
  }
}

// VARLEN: total floats of all stored rows.
__global__ __launch_bounds__(kBlock) void k_sum_lens(const Slot* __restrict__ slots, uint64_t cap,
                                                    const DevState* st,
                                                    unsigned long long* total) {
  unsigned long long s = 0;
  const uint64_t stride = (uint64_t)gridDim.x * kBlock;
  for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < cap; i += stride) {
    const ulonglong2 v = *reinterpret_cast<const ulonglong2*>(&slots[i]);
    if (v.x != kEmptyKey) s += v.y & kLenMask;
  }
  if (blockIdx.x == 0 && threadIdx.x == 0 && st->special_present) s += st->special_payload & kLenMask;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
  if ((threadIdx.x & 63) == 0 && s) atomicAdd(total, s);
}

// Plain streaming copy: one non-temporal 16-byte load and store per lane.
__global__ __launch_bounds__(kBlock) void k_copy(f32x4* __restrict__ dst,
                                                const f32x4* __restrict__ src, uint64_t n16) {
  const uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < n16) __builtin_nontemporal_store(__builtin_nontemporal_load(&src[i]), &dst[i]);
}

}  // namespace pskv
#endif  // PSKV_TABLE_KERNELS_H_
