// Exclusive prefix sum of int32 lens into uint64 offsets in two launches: per-workgroup
// totals (the last workgroup to finish scans them), then a per-workgroup rescan. Used for
// KVWorker::DefaultSlicer's value offsets (include/ps/kv_app.h:563-567) and for
// the request-side row offsets of the var-len store (KVPairs layout, kv_app.h:24-31).
#ifndef PSKV_SCAN_H_
#define PSKV_SCAN_H_
#include "device_common.h"

namespace pskv {

// Lens per thread: 8 for long requests, 1 for short ones so that even 100k lens spread over
// a few hundred workgroups.
constexpr int kScanItemsLarge = 8;
constexpr uint64_t kScanLargeKeys = 1u << 20;

// Sum over the workgroup; result valid in every thread. `red` holds kBlock/64 entries.
__device__ __forceinline__ unsigned long long block_sum_u64(unsigned long long x,
                                                            unsigned long long* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o);
  const unsigned wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[wave] = x;
  __syncthreads();
  unsigned long long t = 0;
#pragma unroll
  for (int w = 0; w < kBlock / 64; ++w) t += red[w];
  return t;
}

// Turns the per-workgroup totals into exclusive offsets, in place. Run by one workgroup.
__device__ __forceinline__ void scan_spine(unsigned long long* __restrict__ part, uint64_t nparts,
                                           unsigned long long* wsum, unsigned long long* carry_s) {
  if (threadIdx.x == 0) *carry_s = 0;
  __syncthreads();
  for (uint64_t base = 0; base < nparts; base += kBlock) {
    const uint64_t i = base + threadIdx.x;
    const unsigned long long x = i < nparts ? part[i] : 0ull;
    const unsigned long long inc = wave_incl_scan_u64(x);
    const unsigned wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 63) wsum[wave] = inc;
    __syncthreads();
    unsigned long long before = *carry_s;
    for (unsigned w = 0; w < wave; ++w) before += wsum[w];
    if (i < nparts) part[i] = before + inc - x;
    __syncthreads();
    if (threadIdx.x == kBlock - 1) *carry_s = before + inc;
    __syncthreads();
  }
}

// Pass 1: per-workgroup totals of the lens; the workgroup that finishes last scans the
// totals (a ticket counter tells it that it is last), so the spine needs no launch of its own.
// Lens are summed as sign-extended 64-bit values modulo 2^64, which is what
// `size_t val_end += int l` does in the reference (kv_app.h:565).
// With a table state `st` the pass also collects two facts about the lens for the row
// kernels (any length not a multiple of 4, any length out of range); the last workgroup
// publishes them as this request's flags and folds the previous request's error bits into
// the sticky ones, which makes it the point where one request's flags end and the next begin.
template <int kScanItems>
__global__ __launch_bounds__(kBlock) void k_scan_partials(const int32_t* __restrict__ lens,
                                                         uint64_t n,
                                                         unsigned long long* __restrict__ part,
                                                         unsigned int* ticket, DevState* st,
                                                         unsigned max_len, ReqTag tag) {
  if (st && cache_same(st, tag)) return;  // offsets and flags of the cached request still hold
  __shared__ unsigned long long red[kBlock / 64];
  __shared__ unsigned long long carry_s;
  __shared__ unsigned s_ticket;
  constexpr int kScanChunk = kBlock * kScanItems;
  const uint64_t base = (uint64_t)blockIdx.x * kScanChunk + (uint64_t)threadIdx.x * kScanItems;
  unsigned long long s = 0;
  unsigned bits = 0, bad = 0;
#pragma unroll
  for (int j = 0; j < kScanItems; ++j) {
    if (base + j < n) {
      const int32_t l = lens[base + j];
      s += (unsigned long long)(long long)l;
      bits |= (unsigned)l & 3u;
      bad |= (l < 0 || (unsigned)l > max_len) ? 1u : 0u;
    }
  }
  const unsigned long long tot = block_sum_u64(s, red);
  if (st) {
    // one atomic per workgroup at most: atomics on one address are served one at a time
    const unsigned b0 = __syncthreads_or(bits & 1u) ? 1u : 0u;
    const unsigned b1 = __syncthreads_or(bits & 2u) ? 2u : 0u;
    const unsigned any_bad = __syncthreads_or(bad) ? 1u : 0u;
    if (threadIdx.x == 0) {
      if (b0 | b1) atomicOr(&st->scan_bits, b0 | b1);
      if (any_bad) atomicOr(&st->scan_bad, 1u);
    }
  }
  if (threadIdx.x == 0) {
    part[blockIdx.x] = tot;
    __threadfence();  // the total (and the flags) before the ticket
    s_ticket = atomicAdd(ticket, 1u);
  }
  __syncthreads();
  if (s_ticket != gridDim.x - 1) return;
  __threadfence();  // see the totals of every other workgroup
  scan_spine(part, gridDim.x, red, &carry_s);
  if (threadIdx.x == 0) {
    *ticket = 0;  // ready for the next scan on this stream
    if (st) {
      st->error |= st->req_error;
      const bool bad_len = atomicExch(&st->scan_bad, 0u) != 0u;
      st->req_error = bad_len ? kDevErrBadLen : 0u;
      if (bad_len) st->bad_epoch = tag.epoch;
      st->misaligned = atomicExch(&st->scan_bits, 0u);
    }
  }
}

// Pass 2: every workgroup rescans its lens from its exclusive offset. With a tile table it
// also records, for each request-side tile of `tile` floats, the key that owns the tile's
// first float: key j owns floats [off[j], off[j+1]), so every tile gets exactly one writer
// and the row kernel needs no search to find where a tile starts. Entry `ntiles` closes it.
template <int kScanItems>
__global__ __launch_bounds__(kBlock) void k_scan_final(const int32_t* __restrict__ lens,
                                                      uint64_t n,
                                                      const unsigned long long* __restrict__ part,
                                                      uint64_t* __restrict__ off, DevState* st,
                                                      uint32_t* __restrict__ tile_key,
                                                      uint64_t ntiles, uint64_t tile, ReqTag tag) {
  if (st && cache_same(st, tag)) return;
  __shared__ unsigned long long wsum[kBlock / 64];
  constexpr int kScanChunk = kBlock * kScanItems;
  const uint64_t base = (uint64_t)blockIdx.x * kScanChunk + (uint64_t)threadIdx.x * kScanItems;
  unsigned long long v[kScanItems];
  unsigned long long s = 0;
#pragma unroll
  for (int j = 0; j < kScanItems; ++j) {
    v[j] = (base + j < n) ? (unsigned long long)(long long)lens[base + j] : 0ull;
    s += v[j];
  }
  const unsigned long long inc = wave_incl_scan_u64(s);
  const unsigned wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 63) wsum[wave] = inc;
  __syncthreads();
  unsigned long long run = part[blockIdx.x] + inc - s;
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
    if (base + j + 1 == n) {  // the thread that owns the last element closes the array
      off[n] = run;
      if (st) st->scan_total = run;
    }
  }
}

inline uint64_t scan_items(uint64_t n) { return n >= kScanLargeKeys ? kScanItemsLarge : 1; }
inline uint64_t scan_num_parts(uint64_t n) {
  const uint64_t chunk = (uint64_t)kBlock * scan_items(n);
  return (n + chunk - 1) / chunk;
}

// off must hold n+1 entries, part scan_num_parts(n) entries, *ticket must be 0 (the scan leaves
// it at 0). n == 0 writes off[0] = 0. tile_key may be nullptr.
inline hipError_t launch_lens_scan(const int32_t* lens, uint64_t n, uint64_t* off,
                                   unsigned long long* part, unsigned int* ticket, DevState* st,
                                   unsigned max_len, uint32_t* tile_key, uint64_t ntiles,
                                   uint64_t tile, ReqTag tag, hipStream_t stream) {
  if (n == 0) return hipMemsetAsync(off, 0, sizeof(uint64_t), stream);
  const uint64_t nparts = scan_num_parts(n);
  const dim3 grid((unsigned)nparts), block(kBlock);
  if (scan_items(n) == kScanItemsLarge) {
    k_scan_partials<kScanItemsLarge><<<grid, block, 0, stream>>>(lens, n, part, ticket, st, max_len, tag);
    k_scan_final<kScanItemsLarge><<<grid, block, 0, stream>>>(lens, n, part, off, st, tile_key, ntiles,
                                                               tile, tag);
  } else {
    k_scan_partials<1><<<grid, block, 0, stream>>>(lens, n, part, ticket, st, max_len, tag);
    k_scan_final<1><<<grid, block, 0, stream>>>(lens, n, part, off, st, tile_key, ntiles, tile, tag);
  }
  return hipGetLastError();
}

}  // namespace pskv
#endif  // PSKV_SCAN_H_
