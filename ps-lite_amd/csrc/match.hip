// Ordered match of two sorted key sets on the GPU (gfx950): the merge-join that the reference
// sketches in ParallelOrderedMatch (include/ps/internal/parallel_kv_match.h:29-120) with the
// operators of assign_op.h:12-41:
//     if (dst_key[i] == src_key[j]) dst_val[i] op= src_val[j]        (k floats per key)
// Both key sets are sorted, so the source keys that can match a tile of destination keys are
// one contiguous stretch. A first small kernel finds where every tile's stretch begins (one
// search per tile, all tiles at once); a workgroup then stages its stretch in LDS and resolves
// its destination keys there, so all key traffic is streamed, once. For k == 1 the values
// are combined in the same kernel; for longer values the kernel leaves the matched source
// index of every destination key behind and a second kernel streams the rows.
#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

#include <mutex>
#include <new>

#include "device_common.h"
#include "host_common.h"

namespace pskv {
namespace {

constexpr unsigned kMatchBlock = 256;
constexpr unsigned kMatchItems = 4;
constexpr unsigned kMatchTile = kMatchBlock * kMatchItems;  // destination keys per workgroup
constexpr unsigned kMatchLds = 2048;    // source keys a workgroup holds in LDS at a time (16 KiB)
constexpr unsigned kMatchPieces = 8;    // a longer stretch than this many pieces is searched in place
constexpr uint64_t kNoMatch = ~0ull;

// first index in [lo, hi) whose key is not below `key`
__device__ __forceinline__ uint64_t lower_bound_of(const uint64_t* __restrict__ a, uint64_t lo, uint64_t hi,
                                                   uint64_t key) {
  while (lo < hi) {
    const uint64_t mid = lo + ((hi - lo) >> 1);
    if (a[mid] < key) lo = mid + 1; else hi = mid;
  }
  return lo;
}

// assign_op.h:26-36: right op= left
__device__ __forceinline__ float combine(int op, float d, float s) {
  switch (op) {
    case PSKV_OP_PLUS: return d + s;
    case PSKV_OP_MINUS: return d - s;
    case PSKV_OP_TIMES: return d * s;
    case PSKV_OP_DIVIDE: return d / s;
    default: return s;
  }
}
__device__ __forceinline__ f32x4 combine(int op, f32x4 d, f32x4 s) {
  f32x4 r;
  r.x = combine(op, d.x, s.x), r.y = combine(op, d.y, s.y);
  r.z = combine(op, d.z, s.z), r.w = combine(op, d.w, s.w);
  return r;
}

// spans[t] = first source key not below the first destination key of tile t; spans[tiles] = n_src.
// The stretch of tile t is [spans[t], spans[t+1]): it may hold source keys that lie between two
// tiles, which match nothing. One wavefront per tile: 64 probes per round narrow the range by a
// factor of 64, so 16M source keys take four dependent loads where halving takes 24.
__global__ __launch_bounds__(kMatchBlock) void k_match_spans(const uint64_t* __restrict__ src, uint64_t n_src,
                                                             const uint64_t* __restrict__ dst, uint64_t tiles,
                                                             uint64_t* __restrict__ spans) {
  const uint64_t t = (uint64_t)blockIdx.x * (kMatchBlock / 64) + (threadIdx.x >> 6);
  const unsigned lane = threadIdx.x & 63;
  if (t > tiles) return;  // (whole wavefronts)
  if (t == tiles) {
    if (lane == 0) spans[t] = n_src;
    return;
  }
  const uint64_t key = dst[t * kMatchTile];
  // every source key before lo is below the key, none from hi on is
  uint64_t lo = 0, hi = n_src;
  while (lo < hi) {
    const uint64_t step = (hi - lo + 63) / 64;
    const uint64_t p = lo + lane * step;
    const bool below = p < hi && src[p] < key;
    const unsigned cnt = (unsigned)__popcll(__ballot(below));  // the probes are sorted: the first cnt are below
    if (cnt == 0) break;
    const uint64_t next = lo + cnt * step;  // the first probe that is not below, if there is one
    lo += (cnt - 1) * step + 1;
    if (cnt < 64 && next < hi) hi = next;
  }
  if (lane == 0) spans[t] = lo;
}

// One workgroup per kMatchTile destination keys. K1: values are single floats and are combined
// here; otherwise where[i] receives the index of the matching source key, or kNoMatch.
template <bool K1>
__global__ __launch_bounds__(kMatchBlock) void k_match_keys(const uint64_t* __restrict__ src, uint64_t n_src,
                                                            const uint64_t* __restrict__ dst, uint64_t n_dst,
                                                            const uint64_t* __restrict__ spans,
                                                            uint64_t* __restrict__ where,
                                                            const float* __restrict__ src_vals,
                                                            float* __restrict__ dst_vals, int op,
                                                            unsigned* __restrict__ tile_count) {
  __shared__ uint64_t s_keys[kMatchLds];
  __shared__ unsigned s_red[kMatchBlock / 64];
  const uint64_t first = (uint64_t)blockIdx.x * kMatchTile;
  const uint64_t tile_n = n_dst - first < kMatchTile ? n_dst - first : kMatchTile;
  // A lane takes kMatchItems neighbouring destination keys (requested before anything else): the
  // first is found by halving, the others a few source keys further on.
  const unsigned idx0 = threadIdx.x * kMatchItems;
  const uint64_t i0 = first + idx0;
  uint64_t key[kMatchItems];
  const bool whole = idx0 + kMatchItems <= tile_n;
  if (whole && (reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
    static_assert(kMatchItems == 4, "two 128-bit loads");
    const u64x2 x = *reinterpret_cast<const u64x2*>(dst + i0);
    const u64x2 y = *reinterpret_cast<const u64x2*>(dst + i0 + 2);
    key[0] = x.x, key[1] = x.y, key[2] = y.x, key[3] = y.y;
  } else {
#pragma unroll
    for (unsigned r = 0; r < kMatchItems; ++r) key[r] = idx0 + r < tile_n ? dst[i0 + r] : 0;
  }
  const uint64_t lo = spans[blockIdx.x], hi = spans[blockIdx.x + 1];
  const uint64_t span = hi > lo ? hi - lo : 0;  // (hi >= lo when the keys are sorted)
  // The stretch goes through LDS in pieces of kMatchLds keys. A key is looked up in the first
  // piece whose last key is not below it (or in the last piece).
  const bool staged = span <= (uint64_t)kMatchLds * kMatchPieces;
  uint64_t j[kMatchItems];
  bool open[kMatchItems];
#pragma unroll
  for (unsigned r = 0; r < kMatchItems; ++r) {
    j[r] = kNoMatch;
    open[r] = idx0 + r < tile_n;
  }
  if (staged) {
    for (uint64_t base = 0; base < span; base += kMatchLds) {
      const unsigned len = span - base < kMatchLds ? (unsigned)(span - base) : kMatchLds;
      const bool last_piece = base + len == span;
      if (base) __syncthreads();  // everyone is done with the piece before
      for (unsigned t = threadIdx.x; t < len; t += kMatchBlock) s_keys[t] = src[lo + base + t];
      __syncthreads();
      const uint64_t top = s_keys[len - 1];
      unsigned pos = 0;     // the lane's open keys are above every source key before this one
      bool on_foot = false;  // whether a key of this lane has been placed in this piece already
#pragma unroll
      for (unsigned r = 0; r < kMatchItems; ++r) {
        if (!open[r] || !(key[r] <= top || last_piece)) continue;
        unsigned at = pos;
        if (on_foot) {
          for (unsigned step = 0; step < 4 && at < len && s_keys[at] < key[r]; ++step) ++at;
        }
        if (at < len && s_keys[at] < key[r]) {  // halve what is left
          unsigned end = len;
          ++at;
          while (at < end) {
            const unsigned mid = (at + end) >> 1;
            if (s_keys[mid] < key[r]) at = mid + 1; else end = mid;
          }
        }
        if (at < len && s_keys[at] == key[r]) j[r] = lo + base + at;
        open[r] = false;
        pos = at;
        on_foot = true;
      }
    }
  } else {  // far more source keys than destination keys here: search the stretch where it lies
    uint64_t from = lo;
#pragma unroll
    for (unsigned r = 0; r < kMatchItems; ++r) {
      if (!open[r]) continue;
      const uint64_t p = lower_bound_of(src, from, hi, key[r]);
      if (p < hi && src[p] == key[r]) j[r] = p;
      from = p;
    }
  }
  unsigned found = 0;
#pragma unroll
  for (unsigned r = 0; r < kMatchItems; ++r) found += j[r] != kNoMatch ? 1u : 0u;
  if (K1) {
    const bool vec = whole && (reinterpret_cast<uintptr_t>(dst_vals) & 15) == 0;
    float d[kMatchItems] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (vec) {
      if (op != PSKV_OP_ASSIGN || (found && found != kMatchItems)) {  // what is combined, or what stays
        const f32x4 v = *reinterpret_cast<const f32x4*>(dst_vals + i0);
        d[0] = v.x, d[1] = v.y, d[2] = v.z, d[3] = v.w;
      }
    } else if (op != PSKV_OP_ASSIGN) {
#pragma unroll
      for (unsigned r = 0; r < kMatchItems; ++r)
        if (j[r] != kNoMatch) d[r] = dst_vals[i0 + r];
    }
#pragma unroll
    for (unsigned r = 0; r < kMatchItems; ++r)
      if (j[r] != kNoMatch) d[r] = combine(op, d[r], src_vals[j[r]]);
    if (vec) {
      if (found) {
        f32x4 v;
        v.x = d[0], v.y = d[1], v.z = d[2], v.w = d[3];
        *reinterpret_cast<f32x4*>(dst_vals + i0) = v;
      }
    } else {
#pragma unroll
      for (unsigned r = 0; r < kMatchItems; ++r)
        if (j[r] != kNoMatch) dst_vals[i0 + r] = d[r];
    }
  } else {
    if (whole) {
      u64x2 x, y;
      x.x = j[0], x.y = j[1], y.x = j[2], y.y = j[3];
      *reinterpret_cast<u64x2*>(where + i0) = x;  // (the workspace is 256-byte aligned)
      *reinterpret_cast<u64x2*>(where + i0 + 2) = y;
    } else {
#pragma unroll
      for (unsigned r = 0; r < kMatchItems; ++r)
        if (idx0 + r < tile_n) where[i0 + r] = j[r];
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) found += __shfl_xor(found, o);
  if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = found;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned total = 0;
    for (unsigned w = 0; w < kMatchBlock / 64; ++w) total += s_red[w];
    tile_count[blockIdx.x] = total;  // (thousands of atomic adds on one counter would take turns)
  }
}

// The matched keys of all tiles: one workgroup of 1024 threads, four loads in flight per thread.
constexpr unsigned kTotalBlock = 1024;
__global__ __launch_bounds__(kTotalBlock) void k_match_total(const unsigned* __restrict__ tile_count, uint64_t tiles,
                                                             unsigned long long* __restrict__ count) {
  __shared__ unsigned long long s_sum[kTotalBlock / 64];
  unsigned long long sum = 0;
  for (uint64_t t = threadIdx.x; t < tiles; t += 4 * kTotalBlock) {
    const unsigned a = tile_count[t];
    const unsigned b = t + kTotalBlock < tiles ? tile_count[t + kTotalBlock] : 0;
    const unsigned c = t + 2 * kTotalBlock < tiles ? tile_count[t + 2 * kTotalBlock] : 0;
    const unsigned d = t + 3 * kTotalBlock < tiles ? tile_count[t + 3 * kTotalBlock] : 0;
    sum += (unsigned long long)a + b + c + d;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
  if ((threadIdx.x & 63) == 0) s_sum[threadIdx.x >> 6] = sum;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long total = 0;
    for (unsigned w = 0; w < kTotalBlock / 64; ++w) total += s_sum[w];
    *count = total;
  }
}

// Rows of kq units (floats, or groups of four floats): dst row i op= src row where[i].
template <typename V>
__global__ __launch_bounds__(kMatchBlock) void k_match_rows(const uint64_t* __restrict__ where, uint64_t n_dst,
                                                            uint64_t kq, const V* __restrict__ src,
                                                            V* __restrict__ dst, int op) {
  const uint64_t total = n_dst * kq;
  const uint64_t stride = (uint64_t)gridDim.x * kMatchBlock;
  for (uint64_t base = (uint64_t)blockIdx.x * kMatchBlock; base < total; base += stride) {
    // one division per workgroup and turn; a lane is at most kMatchBlock units further on
    const uint64_t row0 = base / kq;
    const uint64_t c = base - row0 * kq + threadIdx.x;
    const uint64_t over = kq >= kMatchBlock ? (c >= kq ? 1u : 0u) : (uint64_t)((unsigned)c / (unsigned)kq);
    const uint64_t row = row0 + over, col = c - over * kq;
    if (row >= n_dst) continue;
    const uint64_t j = where[row];
    if (j == kNoMatch) continue;
    const V s = __builtin_nontemporal_load(src + j * kq + col);
    V* p = dst + row * kq + col;
    if (op == PSKV_OP_ASSIGN) {
      __builtin_nontemporal_store(s, p);
    } else {
      __builtin_nontemporal_store(combine(op, __builtin_nontemporal_load(p), s), p);
    }
  }
}

// Per device: a stream, the index workspace and, for host-resident calls, staging room. A call
// holds the lock for its whole duration (calls on one device take turns).
struct MatchCtx {
  std::mutex mu;
  hipStream_t stream = nullptr;
  unsigned long long* count_host = nullptr;  // pinned; the kernel that adds the tiles up writes it
  hipEvent_t ev[4] = {nullptr, nullptr, nullptr, nullptr};  // begin/end of the key kernel and of the row kernel
  struct Buf {
    void* ptr = nullptr;
    size_t cap = 0;
  } where, spans, tile_count, stage[4];
};

int room(MatchCtx::Buf* b, size_t bytes, hipStream_t stream) {
  if (bytes <= b->cap) return PSKV_OK;
  if (b->ptr) {
    PSKV_HIP(hipStreamSynchronize(stream));
    PSKV_HIP(hipFree(b->ptr));
    b->ptr = nullptr;
    b->cap = 0;
  }
  const size_t want = (bytes + (bytes >> 2) + 255) & ~(size_t)255;
  PSKV_HIP(hipMalloc(&b->ptr, want));
  b->cap = want;
  return PSKV_OK;
}

MatchCtx* match_ctx(int device, bool create = true) {
  constexpr int kMaxDevices = 64;
  static std::mutex* mu = new std::mutex();
  static MatchCtx* table[kMaxDevices] = {nullptr};
  if (device < 0 || device >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lk(*mu);
  if (table[device] || !create) return table[device];
  MatchCtx* c = new (std::nothrow) MatchCtx();  // kept until the process ends
  if (!c) return nullptr;
  bool ok = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking) == hipSuccess;
  ok = ok && hipHostMalloc(reinterpret_cast<void**>(&c->count_host), sizeof(unsigned long long),
                           hipHostMallocDefault) == hipSuccess;
  for (int e = 0; ok && e < 4; ++e) ok = hipEventCreate(&c->ev[e]) == hipSuccess;
  if (!ok) {
    (void)hipGetLastError();
    for (int e = 0; e < 4; ++e)
      if (c->ev[e]) (void)hipEventDestroy(c->ev[e]);
    if (c->count_host) (void)hipHostFree(c->count_host);
    if (c->stream) (void)hipStreamDestroy(c->stream);
    delete c;
    return nullptr;
  }
  table[device] = c;
  return c;
}

}  // namespace

// Gives back the workspaces and staging buffers the device's match context has grown to (they
// only grow, and a model-size host-resident call leaves several GiB behind).
int match_trim(int device) {
  MatchCtx* c = match_ctx(device, false);
  if (!c) return PSKV_OK;
  DeviceGuard guard(device);
  if (!guard.ok()) return set_error(PSKV_EHIP, "cannot select device %d", device);
  std::lock_guard<std::mutex> lk(c->mu);
  MatchCtx::Buf* bufs[] = {&c->where, &c->spans, &c->tile_count, &c->stage[0], &c->stage[1], &c->stage[2], &c->stage[3]};
  for (MatchCtx::Buf* b : bufs) {
    if (b->ptr) PSKV_HIP(hipFree(b->ptr));
    b->ptr = nullptr;
    b->cap = 0;
  }
  return PSKV_OK;
}

}  // namespace pskv

using namespace pskv;

extern "C" int pskv_match(int device, const uint64_t* src_keys, size_t n_src, const float* src_vals,
                          const uint64_t* dst_keys, size_t n_dst, float* dst_vals, size_t k, int op,
                          uint64_t* matched, float* kernel_ms, int memkind) {
  clear_error();
  if (matched) *matched = 0;
  if (kernel_ms) kernel_ms[0] = kernel_ms[1] = 0.0f;
  if (op < PSKV_OP_ASSIGN || op > PSKV_OP_DIVIDE)
    return set_error(PSKV_EINVAL, "op %d: only ASSIGN, PLUS, MINUS, TIMES and DIVIDE apply to floats", op);
  if (k == 0) return set_error(PSKV_EINVAL, "k must be at least 1");
  if (memkind != PSKV_MEM_DEVICE && memkind != PSKV_MEM_HOST) return set_error(PSKV_EINVAL, "bad memkind");
  if (n_src == 0 || n_dst == 0) return PSKV_OK;  // parallel_kv_match.h:36
  if (!src_keys || !src_vals || !dst_keys || !dst_vals) return set_error(PSKV_EINVAL, "null buffer");
  if (k > (1ull << 31) || n_src > (1ull << 40) || n_dst > (1ull << 40) ||
      (n_src > n_dst ? n_src : n_dst) > (1ull << 44) / k)  // (2^44 floats: no product below overflows)
    return set_error(PSKV_EINVAL, "sizes beyond what one call handles");
  DeviceGuard guard(device);
  if (!guard.ok()) return set_error(PSKV_EHIP, "cannot select device %d", device);
  MatchCtx* c = match_ctx(device);
  if (!c) return set_error(PSKV_EHIP, "cannot set up the match context of device %d", device);
  std::lock_guard<std::mutex> lk(c->mu);
  hipStream_t st = c->stream;
  const uint64_t* d_src = src_keys;
  const uint64_t* d_dst = dst_keys;
  const float* d_sv = src_vals;
  float* d_dv = dst_vals;
  if (memkind == PSKV_MEM_HOST) {
    const size_t bytes[4] = {n_src * 8, n_dst * 8, n_src * k * 4, n_dst * k * 4};
    const void* from[4] = {src_keys, dst_keys, src_vals, dst_vals};
    for (int b = 0; b < 4; ++b) {
      int rc = room(&c->stage[b], bytes[b], st);
      if (rc) return rc;
      PSKV_HIP(hipMemcpyAsync(c->stage[b].ptr, from[b], bytes[b], hipMemcpyHostToDevice, st));
    }
    d_src = static_cast<const uint64_t*>(c->stage[0].ptr);
    d_dst = static_cast<const uint64_t*>(c->stage[1].ptr);
    d_sv = static_cast<const float*>(c->stage[2].ptr);
    d_dv = static_cast<float*>(c->stage[3].ptr);
  }
  const unsigned blocks = (unsigned)((n_dst + kMatchTile - 1) / kMatchTile);
  {
    int rc = room(&c->spans, ((size_t)blocks + 1) * sizeof(uint64_t), st);
    if (rc) return rc;
  }
  uint64_t* spans = static_cast<uint64_t*>(c->spans.ptr);
  {
    int rc = room(&c->tile_count, (size_t)blocks * sizeof(unsigned), st);
    if (rc) return rc;
  }
  unsigned* tile_count = static_cast<unsigned*>(c->tile_count.ptr);
  hipLaunchKernelGGL(k_match_spans, dim3(blocks / (kMatchBlock / 64) + 1), dim3(kMatchBlock), 0, st, d_src, (uint64_t)n_src,
                     d_dst, (uint64_t)blocks, spans);
  // (a launch can carry events of its own, which read the begin and the end of that very dispatch)
  hipEvent_t e0 = kernel_ms ? c->ev[0] : nullptr, e1 = kernel_ms ? c->ev[1] : nullptr;
  hipEvent_t e2 = kernel_ms ? c->ev[2] : nullptr, e3 = kernel_ms ? c->ev[3] : nullptr;
  if (k == 1) {
    hipExtLaunchKernelGGL(k_match_keys<true>, dim3(blocks), dim3(kMatchBlock), 0, st, e0, e1, 0, d_src, (uint64_t)n_src, d_dst,
                       (uint64_t)n_dst, spans, static_cast<uint64_t*>(nullptr), d_sv, d_dv, op, tile_count);
  } else {
    int rc = room(&c->where, n_dst * sizeof(uint64_t), st);
    if (rc) return rc;
    uint64_t* where = static_cast<uint64_t*>(c->where.ptr);
    hipExtLaunchKernelGGL(k_match_keys<false>, dim3(blocks), dim3(kMatchBlock), 0, st, e0, e1, 0, d_src, (uint64_t)n_src, d_dst,
                       (uint64_t)n_dst, spans, where, d_sv, d_dv, op, tile_count);
    const bool vec = k % 4 == 0 && ((reinterpret_cast<uintptr_t>(d_sv) | reinterpret_cast<uintptr_t>(d_dv)) & 15) == 0;
    const uint64_t kq = vec ? k / 4 : k;
    const unsigned grid = grid_for(n_dst * kq, kMatchBlock, 1u << 20);
    if (vec) {
      hipExtLaunchKernelGGL(k_match_rows<f32x4>, dim3(grid), dim3(kMatchBlock), 0, st, e2, e3, 0, where, (uint64_t)n_dst, kq,
                         reinterpret_cast<const f32x4*>(d_sv), reinterpret_cast<f32x4*>(d_dv), op);
    } else {
      hipExtLaunchKernelGGL(k_match_rows<float>, dim3(grid), dim3(kMatchBlock), 0, st, e2, e3, 0, where, (uint64_t)n_dst, kq, d_sv,
                         d_dv, op);
    }
  }
  hipLaunchKernelGGL(k_match_total, dim3(1), dim3(kTotalBlock), 0, st, tile_count, (uint64_t)blocks, c->count_host);
  PSKV_HIP(hipGetLastError());
  if (memkind == PSKV_MEM_HOST)
    PSKV_HIP(hipMemcpyAsync(dst_vals, d_dv, n_dst * k * 4, hipMemcpyDeviceToHost, st));
  PSKV_HIP(hipStreamSynchronize(st));
  if (matched) *matched = (uint64_t)*static_cast<volatile unsigned long long*>(c->count_host) * k;  // values, not keys (:52)
  if (kernel_ms) {
    PSKV_HIP(hipEventElapsedTime(&kernel_ms[0], c->ev[0], c->ev[1]));
    if (k > 1) PSKV_HIP(hipEventElapsedTime(&kernel_ms[1], c->ev[2], c->ev[3]));
  }
  return PSKV_OK;
}
