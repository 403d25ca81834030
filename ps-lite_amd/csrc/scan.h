// Exclusive prefix sum of int32 lens into uint64 offsets in two passes: per-workgroup
// totals (the last workgroup to finish scans them), then a per-workgroup rescan. These are
// the building blocks; the kernels of the var-len store (table_kernels.h) run pass 1 in the
// kernel that first touches a request's lens and pass 2 in the kernel that follows, so the
// scan costs no launch of its own. The offsets are the request-side row offsets of the
// KVPairs layout (include/ps/kv_app.h:24-31).
#ifndef PSKV_SCAN_H_
#define PSKV_SCAN_H_
#include "device_common.h"

namespace pskv {

// Keys per thread: 4 for long requests (fewer atomic adds on the arena counter and fewer
// tickets), 1 for short ones so that even 100k keys spread over a few hundred workgroups.
constexpr int kScanItemsLarge = 4;
constexpr uint64_t kScanLargeKeys = 1u << 20;

// Sum of `x` and OR of `f` over the workgroup; results valid in every thread. `red` and
// `fred` hold kBlock/64 entries each.
__device__ __forceinline__ void block_sum_or(unsigned long long& x, unsigned& f,
                                             unsigned long long* red, unsigned* fred) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    x += __shfl_xor(x, o);
    f |= __shfl_xor(f, o);
  }
  const unsigned wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) {
    red[wave] = x;
    fred[wave] = f;
  }
  __syncthreads();
  unsigned long long t = 0;
  unsigned g = 0;
#pragma unroll
  for (int w = 0; w < kBlock / 64; ++w) {
    t += red[w];
    g |= fred[w];
  }
  x = t;
  f = g;
}

// Turns the per-workgroup totals into exclusive offsets, in place, and leaves the grand total
// in *carry_s. Run by one workgroup. Every thread takes kSpineItems consecutive totals, so
// up to kBlock*kSpineItems of them cost one round of loads and one of stores.
constexpr int kSpineItems = 16;
__device__ __forceinline__ void scan_spine(unsigned long long* part, uint64_t nparts,
                                           unsigned long long* wsum, unsigned long long* carry_s) {
  if (threadIdx.x == 0) *carry_s = 0;
  __syncthreads();
  for (uint64_t base = 0; base < nparts; base += (uint64_t)kBlock * kSpineItems) {
    const uint64_t first = base + (uint64_t)threadIdx.x * kSpineItems;
    unsigned long long x[kSpineItems];
    unsigned long long mine = 0;
#pragma unroll
    for (int j = 0; j < kSpineItems; ++j) {
      x[j] = first + j < nparts ? part[first + j] : 0ull;
      mine += x[j];
    }
    const unsigned long long inc = wave_incl_scan_u64(mine);
    const unsigned wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 63) wsum[wave] = inc;
    __syncthreads();
    unsigned long long run = *carry_s + inc - mine;
    for (unsigned w = 0; w < wave; ++w) run += wsum[w];
#pragma unroll
    for (int j = 0; j < kSpineItems; ++j) {
      if (first + j < nparts) part[first + j] = run;
      run += x[j];
    }
    __syncthreads();
    if (threadIdx.x == kBlock - 1) *carry_s = run;
    __syncthreads();
  }
}

// Pass 1, the workgroup's part. Every thread calls it with the sum of its lens, taken as
// sign-extended 64-bit values modulo 2^64 (what `size_t val_end += int l` does in the
// reference, kv_app.h:565), and the kReq* facts it found. The workgroup's total goes to
// part[blockIdx.x], its facts to DevState::req_flags (one atomic per workgroup at most).
// Returns true in every thread of the workgroup that finishes last of the `nblk` that scan this
// table's request. `red`/`fred` hold kBlock/64 words each.
__device__ __forceinline__ bool scan_pass1_block(unsigned long long s, unsigned flags,
                                                 unsigned long long* __restrict__ part,
                                                 DevState* st, unsigned nblk,
                                                 unsigned long long* red, unsigned* fred,
                                                 unsigned* s_last) {
  block_sum_or(s, flags, red, fred);
  if (threadIdx.x == 0) {
    if (flags) atomicOr(&st->req_flags, flags);
    publish_u64(&part[blockIdx.x], s);
    *s_last = ticket_last(st, nblk) ? 1u : 0u;
  }
  __syncthreads();
  return *s_last != 0u;
}

// Pass 1, what the last workgroup does once all totals are there: it turns them into
// exclusive offsets in place, stores the grand total, publishes the request's flags and folds
// the previous request's error bits into the sticky ones, which makes this the point where
// one request's flags end and the next begin. Every thread of that workgroup calls it;
// the facts collected from all workgroups are returned in thread 0.
__device__ __forceinline__ unsigned scan_pass1_last(unsigned long long* part, DevState* st,
                                                    unsigned nblk, unsigned long long epoch,
                                                    unsigned long long* red,
                                                    unsigned long long* carry_s) {
  scan_spine(part, nblk, red, carry_s);
  unsigned flags = 0;
  if (threadIdx.x == 0) {
    flags = atomicExch(&st->req_flags, 0u);
    st->scan_total = *carry_s;
    st->error |= st->req_error;
    const bool bad_len = (flags & kReqBadLen) != 0u;
    const bool dup = (flags & kReqDuplicate) != 0u;
    st->req_error = (bad_len ? kDevErrBadLen : 0u) | (dup ? kDevErrDuplicate : 0u);
    if (bad_len || dup) st->bad_epoch = epoch;
    st->misaligned = flags & kReqMisaligned;
  }
  return flags;
}

// Pass 2, the workgroup's part: every thread passes its kScanItems consecutive lens
// (sign-extended; zero past the end) starting at index `base`; the workgroup rescans them from
// its exclusive offset `part_b` and writes off[]. With a tile table it also records, for each
// request-side tile of `tile` floats, the key that owns the tile's first float: key j owns
// floats [off[j], off[j+1]), so every tile gets exactly one writer and the row kernel needs no
// search to find where a tile starts. Entry `ntiles` closes the table. `wsum` holds kBlock/64
// words.
template <int kScanItems>
__device__ __forceinline__ void scan_pass2_offsets(const unsigned long long (&v)[kScanItems],
                                                   uint64_t base, uint64_t n,
                                                   unsigned long long part_b,
                                                   uint64_t* __restrict__ off,
                                                   uint32_t* __restrict__ tile_key, uint64_t ntiles,
                                                   uint64_t tile, unsigned long long* wsum) {
  unsigned long long s = 0;
#pragma unroll
  for (int j = 0; j < kScanItems; ++j) s += v[j];
  const unsigned long long inc = wave_incl_scan_u64(s);
  const unsigned wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 63) wsum[wave] = inc;
  __syncthreads();
  unsigned long long run = part_b + inc - s;
  for (unsigned w = 0; w < wave; ++w) run += wsum[w];
  if (tile_key && base == 0) tile_key[ntiles] = (uint32_t)(n - 1);
#pragma unroll
  for (int j = 0; j < kScanItems; ++j) {
    if (base + j < n) {
      off[base + j] = run;
      const unsigned long long end = run + v[j];
      // only sane lens reach here with a tile table (the row kernels refuse the others)
      if (tile_key && end > run && v[j] <= 0xffffffffull) {
        uint64_t t = (run + tile - 1) / tile;
        const uint64_t t_last = (end - 1) / tile;
        for (; t <= t_last && t < ntiles; ++t) tile_key[t] = (uint32_t)(base + j);
      }
    }
    run += v[j];
    if (base + j + 1 == n) off[n] = run;  // the thread that owns the last element closes the array
  }
}

// `n_largest`: the longest key list among the tables a launch serves; all of them use one split.
inline int scan_items(uint64_t n_largest) { return n_largest >= kScanLargeKeys ? kScanItemsLarge : 1; }
inline uint64_t scan_num_parts(uint64_t n, int items) {
  const uint64_t chunk = (uint64_t)kBlock * items;
  return (n + chunk - 1) / chunk;
}

}  // namespace pskv
#endif  // PSKV_SCAN_H_
