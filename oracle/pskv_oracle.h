/*
 * CPU oracle for the ps-lite server-side key-value data path.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing that ships may call into this library:
 * it exists so that tests, the smoke check and the benchmark's cpu_baseline
 * leg can compare the HIP path against a plain single-threaded restatement
 * of what the reference computes.
 *
 * Every entry point names the reference lines it restates. Functions marked
 * "extended" have no counterpart in the reference (its default handle only
 * stores one value per key); their rules are the ones this build froze and
 * they are pinned by reduction to the scalar case, closed forms and numpy.
 *
 * Pinning status (what the CPU test-suite checks each function against):
 *   pskv_oracle_server_ranges  recorded outputs of the reference for S=4, closed form
 *   pskv_oracle_slice          numpy.searchsorted / cumsum, brute force, recorded
 *                              reference outputs, and the real DefaultSlicer when
 *                              oracle/_ref is built
 *   pskv_oracle_handle scalar  dict-of-float32 model, closed forms of
 *                              tests/test_kv_app.cc:53-60, recorded reference outputs
 *   pskv_oracle_handle fixed-k / var-len (extended)
 *                              k=1 equals scalar, numpy row sums, closed forms
 *   pskv_oracle_assemble_pull  numpy concatenation after argsort, FindRange doc example
 *   pskv_oracle_ordered_match  (the reference's header does not compile, so there is no build
 *                              of it to compare with) numpy searchsorted model, closed forms:
 *                              equal key sets, disjoint key sets, one-sided subsets, k > 1
 */
#ifndef PSKV_ORACLE_H_
#define PSKV_ORACLE_H_
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* status codes: identical numbering to include/pskv/capi.h */
#define PSKV_ORACLE_OK 0
#define PSKV_ORACLE_EUNCOVERED_KEY (-1) /* kv_app.h:542 CHECK_EQ(pos[n], keys.size()) */
#define PSKV_ORACLE_ESIZE_MISMATCH (-2) /* kv_app.h:447,489,549,551; sarray.h:249 */
#define PSKV_ORACLE_ENOMEM (-3)
#define PSKV_ORACLE_EINVAL (-5)
#define PSKV_ORACLE_ERANGE_GAP (-6)    /* kv_app.h:533 */
#define PSKV_ORACLE_ELEN_CHANGED (-7)  /* extended rule: row length differs from stored */

#define PSKV_ORACLE_MODE_SCALAR 0
#define PSKV_ORACLE_MODE_FIXED 1
#define PSKV_ORACLE_MODE_VARLEN 2

/* Postoffice::GetServerKeyRanges, src/postoffice.cc:169-180:
 * range i = [kMaxKey/S*i, kMaxKey/S*(i+1)), kMaxKey = 2^64-1 (include/ps/base.h:18). */
void pskv_oracle_server_ranges(uint64_t num_servers, uint64_t* begin, uint64_t* end);

/* KVWorker::DefaultSlicer, include/ps/kv_app.h:517-572.
 * keys[n] sorted unique; lens == NULL means "send.lens.empty()".
 * Outputs: pos[S+1] key offsets (kv_app.h:525-541); val_pos[S+1] so that slice i
 * holds vals [val_pos[i], val_pos[i+1]) (kv_app.h:563-570); used[S] = slice.first.
 * On a failed CHECK the matching negative status is returned and the outputs
 * written so far are unspecified. */
int pskv_oracle_slice(const uint64_t* keys, size_t n, const int32_t* lens, size_t nlens,
                      size_t nvals, const uint64_t* range_begin, const uint64_t* range_end,
                      size_t S, uint64_t* pos, uint64_t* val_pos, uint8_t* used);

typedef struct pskv_oracle_store pskv_oracle_store;

/* mode SCALAR restates KVServerDefaultHandle's store (kv_app.h:462).
 * FIXED (row_len floats per key; 0 = take it from the first push) and VARLEN are
 * the extended stores. */
pskv_oracle_store* pskv_oracle_store_create(int mode, uint64_t row_len);
void pskv_oracle_store_destroy(pskv_oracle_store* s);

/* One invocation of the request handle, kv_app.h:442-461 (scalar) or its
 * extension. push/pull are KVMeta::push / KVMeta::pull. For a pull the response
 * values are written to out_vals (capacity out_cap floats) and, in VARLEN mode,
 * the response lens to out_lens[n]; *out_nvals receives the number of response
 * floats. If out_cap is too small the status is ESIZE_MISMATCH, *out_nvals
 * holds the needed size and the store is left as if the call had completed
 * (pull-inserts included). */
int pskv_oracle_handle(pskv_oracle_store* s, int push, int pull, const uint64_t* keys, size_t n,
                       const float* vals, size_t nvals, const int32_t* lens, size_t nlens,
                       float* out_vals, size_t out_cap, int32_t* out_lens, size_t* out_nvals);

/* number of keys held (unordered_map::size()) */
size_t pskv_oracle_store_size(const pskv_oracle_store* s);
/* total floats held */
size_t pskv_oracle_store_nvals(const pskv_oracle_store* s);

/* Sorted-by-key dump for stored-key parity. keys[cap_keys], lens[cap_keys] (may be
 * NULL), vals[cap_vals]; *n_keys / *n_vals receive the counts (also when too small,
 * in which case ESIZE_MISMATCH is returned and nothing is written). */
int pskv_oracle_store_dump(const pskv_oracle_store* s, uint64_t* keys, int32_t* lens,
                           size_t cap_keys, float* vals, size_t cap_vals, size_t* n_keys,
                           size_t* n_vals);

/* Worker-side pull reassembly, the callback built by KVWorker::AddPullCB,
 * kv_app.h:663-714: per-server responses (in arrival order) are checked against the
 * request keys with FindRange (sarray.h:281-287), sorted by first key and
 * concatenated. resp_keys/resp_vals/resp_lens are arrays of R pointers, with
 * resp_nkeys/resp_nvals their sizes; resp_lens may be NULL (no lens asked for). */
int pskv_oracle_assemble_pull(const uint64_t* req_keys, size_t n, size_t R,
                              const uint64_t* const* resp_keys, const size_t* resp_nkeys,
                              const float* const* resp_vals, const size_t* resp_nvals,
                              const int32_t* const* resp_lens, float* out_vals, size_t out_cap,
                              int32_t* out_lens, size_t* out_nvals);

/* FindRange, include/ps/sarray.h:281-287: index range of keys within [lower, upper). */
void pskv_oracle_find_range(const uint64_t* arr, size_t n, uint64_t lower, uint64_t upper,
                            uint64_t* begin, uint64_t* end);

/* ParallelOrderedMatch, include/ps/internal/parallel_kv_match.h:29-120: for sorted unique keys,
 * dst_vals[i*k .. i*k+k) op= src_vals[j*k .. j*k+k) wherever dst_keys[i] == src_keys[j]; other
 * destination values stay. op: 0 ASSIGN, 1 PLUS, 2 MINUS, 3 TIMES, 4 DIVIDE (assign_op.h:12-21).
 * *matched = k * matched keys (:52). */
int pskv_oracle_ordered_match(const uint64_t* src_keys, size_t n_src, const float* src_vals,
                              const uint64_t* dst_keys, size_t n_dst, float* dst_vals, size_t k,
                              int op, size_t* matched);

#ifdef __cplusplus
}
#endif
#endif /* PSKV_ORACLE_H_ */
