// Exclusive prefix sum of int32 lens into uint64 offsets, three plain launches
// (per-workgroup totals, scan of the totals, per-workgroup rescan). Used for
// KVWorker::DefaultSlicer's value offsets (include/ps/kv_app.h:563-567) and for
// the request-side row offsets of the var-len store (KVPairs layout, kv_app.h:24-31).
#ifndef PSKV_SCAN_H_
#define PSKV_SCAN_H_
#include "device_common.h"

namespace pskv {

constexpr int kScanItems = 8;                        // lens per thread
constexpr int kScanChunk = kBlock * kScanItems;      // lens per workgroup

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

// Lens are summed as sign-extended 64-bit values modulo 2^64, which is what
// `size_t val_end += int l` does in the reference (kv_app.h:565).
__global__ __launch_bounds__(kBlock) void k_scan_partials(const int32_t* __restrict__ lens,
                                                         uint64_t n,
                                                         unsigned long long* __restrict__ part,
                                                         DevState* st, unsigned max_len) {
  __shared__ unsigned long long red[kBlock / 64];
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
  if (threadIdx.x == 0) part[blockIdx.x] = tot;
  if (st) {
    if (bits) atomicOr(&st->misaligned, bits);
    if (bad) atomicOr(&st->error, kDevErrBadLen);
  }
}

// One workgroup turns the per-workgroup totals into exclusive offsets, in place.
__global__ __launch_bounds__(kBlock) void k_scan_spine(unsigned long long* __restrict__ part,
                                                      uint64_t nparts) {
  __shared__ unsigned long long wsum[kBlock / 64];
  __shared__ unsigned long long carry_s;
  if (threadIdx.x == 0) carry_s = 0;
  __syncthreads();
  for (uint64_t base = 0; base < nparts; base += kBlock) {
    const uint64_t i = base + threadIdx.x;
    const unsigned long long x = i < nparts ? part[i] : 0ull;
    const unsigned long long inc = wave_incl_scan_u64(x);
    const unsigned wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 63) wsum[wave] = inc;
    __syncthreads();
    unsigned long long before = carry_s;
    for (unsigned w = 0; w < wave; ++w) before += wsum[w];
    if (i < nparts) part[i] = before + inc - x;
    __syncthreads();
    if (threadIdx.x == kBlock - 1) carry_s = before + inc;
    __syncthreads();
  }
}

__global__ __launch_bounds__(kBlock) void k_scan_final(const int32_t* __restrict__ lens,
                                                      uint64_t n,
                                                      const unsigned long long* __restrict__ part,
                                                      uint64_t* __restrict__ off, DevState* st) {
  __shared__ unsigned long long wsum[kBlock / 64];
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
#pragma unroll
  for (int j = 0; j < kScanItems; ++j) {
    if (base + j < n) off[base + j] = run;
    run += v[j];
    if (base + j + 1 == n) {  // the thread that owns the last element closes the array
      off[n] = run;
      if (st) st->scan_total = run;
    }
  }
}

inline uint64_t scan_num_parts(uint64_t n) { return (n + kScanChunk - 1) / kScanChunk; }

// off must hold n+1 entries, part scan_num_parts(n) entries. n == 0 writes off[0] = 0.
inline hipError_t launch_lens_scan(const int32_t* lens, uint64_t n, uint64_t* off,
                                   unsigned long long* part, DevState* st, unsigned max_len,
                                   hipStream_t stream) {
  if (n == 0) {
    hipError_t e = hipMemsetAsync(off, 0, sizeof(uint64_t), stream);
    return e;
  }
  const uint64_t nparts = scan_num_parts(n);
  k_scan_partials<<<dim3((unsigned)nparts), dim3(kBlock), 0, stream>>>(lens, n, part, st, max_len);
  k_scan_spine<<<dim3(1), dim3(kBlock), 0, stream>>>(part, nparts);
  k_scan_final<<<dim3((unsigned)nparts), dim3(kBlock), 0, stream>>>(lens, n, part, off, st);
  return hipGetLastError();
}

}  // namespace pskv
#endif  // PSKV_SCAN_H_
