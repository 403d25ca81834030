/*
 * pskv C ABI: the MI355X (gfx950) server-side key-value data path of a
 * ps-lite style parameter server, as a plain-C boundary.
 *
 * What sits behind it: an open-addressing hash table resident in HBM
 * (find-or-insert + accumulate on push, gather on pull), row accumulation for
 * fixed-length and variable-length values, and the worker-side key-range
 * slicer (boundary search + lens scan). All kernels are HIP for gfx950.
 *
 * Conventions
 *  - Every function returns an int status: 0 on success, a negative PSKV_E*
 *    code otherwise; pskv_last_error() gives the text for the calling thread.
 *    Nothing throws across this boundary.
 *  - `memkind` says where the caller's buffers live. PSKV_MEM_DEVICE pointers
 *    are device memory on the table's device and are used in place;
 *    PSKV_MEM_HOST pointers are ordinary host memory and are staged through
 *    pinned buffers owned by the library.
 *  - Calls with PSKV_MEM_DEVICE buffers are asynchronous: work is enqueued on
 *    the table's stream in call order and the caller's buffers must stay valid
 *    until pskv_sync(). Input buffers written by other streams must be complete
 *    before the call. Calls with PSKV_MEM_HOST buffers return when the caller's
 *    buffers are the caller's again: inputs have been read, responses are in place.
 *    (A pure push of a PSKV_MODE_SCALAR table of up to 128 KiB of keys and values, about
 *    10,000 keys, has nothing to hand back and returns once its input has been copied to
 *    pinned memory and its kernel is queued; up to eight such pushes are in flight at a
 *    time, later requests follow them in call order, pskv_sync() waits for them.)
 *  - Keys within one request must be unique (ps-lite requires sorted unique
 *    keys, include/ps/kv_app.h:17); requests on one table are applied in call
 *    order. A SORTED request that repeats a key: the row modes refuse it as a whole with
 *    PSKV_EINVAL (no stored value changes; PSKV_MODE_FIXED may leave the keys it named as
 *    zero rows, as a pull of them would), PSKV_MODE_SCALAR gives the result of the
 *    reference's loop (kv_app.h:451-459). An unsorted request that repeats a key has an
 *    unspecified result in every mode (no memory other than its keys' values is touched).
 *    A table must not be used from two threads at once (the reference
 *    runs the handle on one Customer thread, src/customer.cc:49-63).
 *    pskv_slice is re-entrant.
 *
 * Reference lines are relative to the root of dmlc/ps-lite.
 */
#ifndef PSKV_CAPI_H_
#define PSKV_CAPI_H_
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PSKV_OK 0
#define PSKV_EUNCOVERED_KEY (-1) /* a key lies beyond the last range: kv_app.h:542 */
#define PSKV_ESIZE_MISMATCH (-2) /* kv_app.h:447,489,549,551; sarray.h:249; output too small */
#define PSKV_ENOMEM (-3)
#define PSKV_EHIP (-4)           /* a HIP runtime call failed */
#define PSKV_EINVAL (-5)
#define PSKV_ERANGE_GAP (-6)     /* ranges[i-1].end != ranges[i].begin: kv_app.h:533 */
#define PSKV_ELEN_CHANGED (-7)   /* var-len push with a length that differs from the stored row */
#define PSKV_ESTALE (-8)         /* a recorded request (pskv_replay_*) no longer fits its tables or its keys */

#define PSKV_MEM_HOST 0
#define PSKV_MEM_DEVICE 1

#define PSKV_MODE_SCALAR 0 /* one float per key: KVServerDefaultHandle, kv_app.h:440-463 */
#define PSKV_MODE_FIXED 1  /* k floats per key, k = vals/keys: KVPairs layout kv_app.h:17-22 */
#define PSKV_MODE_VARLEN 2 /* lens[i] floats per key: KVPairs layout kv_app.h:24-31 */

/* longest row a PSKV_MODE_VARLEN table stores, in floats */
#define PSKV_MAX_VARLEN_ROW ((1u << 28) - 1)

/* kernels whose device time pskv_prof_read reports */
#define PSKV_KERNEL_PUSH_SCALAR 0
#define PSKV_KERNEL_PULL_SCALAR 1
#define PSKV_KERNEL_ROWS_ACC 2    /* push accumulate of rows (fixed-k and var-len) */
#define PSKV_KERNEL_ROWS_GATHER 3 /* pull gather of rows */
#define PSKV_KERNEL_LOOKUP 4      /* key -> row lookup / insert of the row modes */
#define PSKV_KERNEL_REHASH 5
#define PSKV_KERNEL_COPY 6        /* the plain copy of pskv_copy_probe */
#define PSKV_KERNEL_SAME_KEYS 7   /* comparison of a request's keys with the cached key set */
#define PSKV_KERNEL_PULL_PER_KEY 8 /* SCALAR pull right behind the push that filled the key cache: keys
                                     compared and values answered in one pass (booked by a launch's first table) */
#define PSKV_KERNEL_COUNT 9

typedef struct pskv_table pskv_table;

typedef struct pskv_opts {
  int32_t device;            /* HIP device ordinal */
  int32_t mode;              /* PSKV_MODE_* */
  uint64_t initial_capacity; /* keys the table should hold before its first growth; 0 = default */
  uint64_t row_len;          /* PSKV_MODE_FIXED: floats per key, 0 = taken from the first push */
  uint64_t arena_floats;     /* row modes: initial value storage in floats, 0 = default */
  float max_load;            /* the fill the slot array is kept below, 0 = 0.5 (a table whose requests have
                                mostly been naming keys it holds may run up to 0.85 rather than grow for the
                                keys of requests in flight that are unlikely to be new) */
  uint32_t reserved;
  void* stream;              /* hipStream_t to run on, NULL = the table creates its own */
} pskv_opts;

/* Replaces the construction of KVServerDefaultHandle and its std::unordered_map
 * store (kv_app.h:441,462; tests/test_kv_app.cc:10-11). */
int pskv_table_create(pskv_table** out, const pskv_opts* opts);
int pskv_table_destroy(pskv_table* t);

/* Push half of the request handle: `store[keys[i]] += vals[i]` with an absent
 * key starting from 0 (kv_app.h:444-455). lens is NULL unless the table is
 * PSKV_MODE_VARLEN (then nlens must equal n, kv_app.h:489). */
int pskv_push(pskv_table* t, const uint64_t* keys, size_t n, const float* vals, size_t nvals,
              const int32_t* lens, size_t nlens, int memkind);

/* Pull half of the request handle: `out[i] = store[keys[i]]`, where an absent key
 * is inserted with value 0 (kv_app.h:448-450,456-458). Row modes write the rows
 * back to back in request order; PSKV_MODE_VARLEN also writes out_lens[n] and
 * answers an absent key with length 0 without inserting it. If the response
 * does not fit out_cap floats the status is PSKV_ESIZE_MISMATCH and *out_nvals
 * (a host pointer, may be NULL) holds the needed size; out/out_lens are then
 * unspecified. In PSKV_MODE_VARLEN the response size is data dependent: with a non-NULL
 * out_nvals the call waits for the device even with PSKV_MEM_DEVICE buffers; with
 * out_nvals == NULL it stays asynchronous, out must have room for the whole response,
 * and a response that does not fit writes nothing and is reported by the next
 * pskv_sync as PSKV_ESIZE_MISMATCH. */
int pskv_pull(pskv_table* t, const uint64_t* keys, size_t n, float* out, size_t out_cap,
              int32_t* out_lens, size_t* out_nvals, int memkind);

/* A request with push and pull both set: per key the push is applied first,
 * then the value is read back (kv_app.h:451-459). */
int pskv_pushpull(pskv_table* t, const uint64_t* keys, size_t n, const float* vals, size_t nvals,
                  const int32_t* lens, size_t nlens, float* out, size_t out_cap,
                  int32_t* out_lens, size_t* out_nvals, int memkind);

/* One process, several logical servers on one GPU. KVWorker::Send turns a sliced request into
 * one message per server range (kv_app.h:590-612); when the tables of those ranges live in one
 * process on one GPU, the calls below serve all of them with ONE launch per step of the
 * pipeline instead of one per table (a launch over 1/S of a request leaves most of the GPU
 * idle). pos[S+1] and val_pos[S+1] are HOST arrays, exactly what pskv_slice returns: slice s
 * holds keys [pos[s], pos[s+1]) and vals [val_pos[s], val_pos[s+1]) (and lens [pos[s],
 * pos[s+1]) in PSKV_MODE_VARLEN) and goes to tables[s]; a slice without keys is skipped, as
 * Send skips it (`first == false`, kv_app.h:581-595). The result is what S calls of pskv_push /
 * pskv_pull would give. The tables must share a device, a mode and a STREAM: create the first,
 * then pass pskv_table_stream(first) as pskv_opts.stream of the others. keys/vals/lens/out/
 * out_lens are device memory (PSKV_MEM_DEVICE is the only memkind accepted) and the calls are
 * asynchronous like the single-table ones. Everything the host can check is checked for all
 * slices before anything is enqueued; device-detected errors are reported per table by
 * pskv_sync / pskv_sync_multi. More than 16 slices with keys are served 16 at a time. */
void* pskv_table_stream(pskv_table* t);
int pskv_push_multi(pskv_table* const* tables, size_t S, const uint64_t* keys, const uint64_t* pos,
                    const float* vals, const uint64_t* val_pos, const int32_t* lens, int memkind);
/* Slice s answers into out[out_pos[s] .. out_pos[s+1]) (room, not necessarily all used) and, in
 * PSKV_MODE_VARLEN, out_lens[pos[s] .. pos[s+1]). out_pos == NULL means out_pos[s] = pos[s] * k
 * (SCALAR: k = 1, FIXED: the row length); PSKV_MODE_VARLEN needs out_pos. A SCALAR/FIXED slice
 * whose room is too small fails the call with PSKV_ESIZE_MISMATCH before anything is enqueued.
 * out_nvals (host array of S, may be NULL) receives the floats each slice answered; in
 * PSKV_MODE_VARLEN a non-NULL out_nvals makes the call wait for the device (and a slice that
 * does not fit fails it with PSKV_ESIZE_MISMATCH, the needed sizes in out_nvals), with NULL it
 * stays asynchronous and a slice that does not fit writes nothing and is reported by the next
 * sync, as in pskv_pull. */
int pskv_pull_multi(pskv_table* const* tables, size_t S, const uint64_t* keys, const uint64_t* pos,
                    float* out, const uint64_t* out_pos, int32_t* out_lens, uint64_t* out_nvals,
                    int memkind);
/* A request with push and pull both set (kv_app.h:451-459) over all slices at once: what S calls of
 * pskv_pushpull would give, arguments as in the two calls above. In PSKV_MODE_VARLEN the call waits for
 * the device between the two halves, as pskv_pushpull does (a refused push is not followed by its pull). */
int pskv_pushpull_multi(pskv_table* const* tables, size_t S, const uint64_t* keys, const uint64_t* pos,
                        const float* vals, const uint64_t* val_pos, const int32_t* lens, float* out,
                        const uint64_t* out_pos, int32_t* out_lens, uint64_t* out_nvals, int memkind);
/* pskv_sync for all tables of a group with one wait: returns the first deferred error (every
 * table's error state is cleared). */
int pskv_sync_multi(pskv_table* const* tables, size_t S);

/* A request that repeats, recorded once and replayed with ONE call. The reference's own test
 * pushes the same keys over and over (tests/test_kv_app.cc:36-44), and so does a worker that
 * trains a dense model: per step KVWorker::Send delivers the same keys in the same slices
 * (kv_app.h:574-613) and only the values differ. pskv_replay_record serves such a request once,
 * exactly as pskv_push_multi (what = PSKV_REPLAY_PUSH), pskv_pull_multi (PSKV_REPLAY_PULL) or
 * the one followed by the other (PSKV_REPLAY_PUSH | PSKV_REPLAY_PULL; PSKV_MODE_SCALAR tables serve
 * the two as one request with both halves, which gives the same values) would, with the same
 * arguments (device memory only; out_vals, out_pos and out_lens as pskv_pull_multi's out,
 * out_pos and out_lens; a PSKV_MODE_VARLEN response that does not fit is reported by the next
 * sync), waits for it, and keeps the launches that a repeat of it takes as a HIP graph on the
 * tables' stream (which must not be the null stream), or, with PSKV_REPLAY_LAUNCHES, as the
 * launches themselves. It allocates and waits; it is a set-up call.
 * pskv_replay_run enqueues that graph (makes those launches again): the request is applied
 * again, to whatever the value buffers hold by the time the stream gets to it (keys, lens, positions and addresses are part
 * of the recording). It allocates nothing, waits for nothing and reads nothing back: the host
 * side of a step is this one call.
 * A replay creates no key and moves no buffer, and the host sizes nothing for it. The device
 * therefore checks first, table by table, that the key (and lens) buffers still hold what was
 * recorded; a table whose slice has changed is left as it is by that run, its part of a pull
 * is not written, and the next pskv_sync / pskv_sync_multi reports PSKV_ESTALE for it.
 * A PSKV_MODE_VARLEN pull on its own can only be recorded right behind a push of the same keys (a
 * var-len pull creates nothing and leaves no key cache behind; PSKV_ESTALE otherwise).
 * Any other request on one of the tables (pskv_push, pskv_pull, pskv_dump, another recording)
 * may move what the recording points at, so it ends the recording's life: pskv_replay_run then
 * returns PSKV_ESTALE and enqueues nothing; record again. pskv_sync, pskv_sync_multi and
 * pskv_size may be called between runs. Destroy a recording before its tables. */
typedef struct pskv_replay pskv_replay;
#define PSKV_REPLAY_PUSH 1
#define PSKV_REPLAY_PULL 2
/* or-ed into `what`: keep the launches themselves instead of a graph; pskv_replay_run then makes them
 * again one by one (same kernels, same arguments, same checks on the device). */
#define PSKV_REPLAY_LAUNCHES 4
int pskv_replay_record(pskv_replay** out, pskv_table* const* tables, size_t S, int what, const uint64_t* keys,
                       const uint64_t* pos, const float* vals, const uint64_t* val_pos, const int32_t* lens,
                       float* out_vals, const uint64_t* out_pos, int32_t* out_lens);
int pskv_replay_run(pskv_replay* r);
int pskv_replay_destroy(pskv_replay* r);

/* Waits for everything enqueued on the table and reports a deferred device-side
 * error (PSKV_ELEN_CHANGED) of an earlier asynchronous push, once. */
int pskv_sync(pskv_table* t);

/* Number of keys held: unordered_map::size() of the reference store (kv_app.h:462).
 * Waits for the device. */
int pskv_size(pskv_table* t, uint64_t* n_keys, uint64_t* n_vals);

/* All stored pairs sorted by key, for stored-key parity checks (the reference has
 * no such call; it is the equivalent of iterating the store, kv_app.h:462).
 * Host buffers only. lens may be NULL. Too small a buffer gives
 * PSKV_ESIZE_MISMATCH with the needed sizes in *n_keys / *n_vals. */
int pskv_dump(pskv_table* t, uint64_t* keys, int32_t* lens, size_t cap_keys, float* vals,
              size_t cap_vals, size_t* n_keys, size_t* n_vals);

/* KVWorker::DefaultSlicer (kv_app.h:517-572): partitions sorted keys over S
 * contiguous key ranges [range_begin[i], range_end[i]) (host arrays, as returned by
 * Postoffice::GetServerKeyRanges, src/postoffice.cc:169-180).
 * Outputs are host arrays: pos[S+1] so that slice i holds keys [pos[i], pos[i+1]),
 * val_pos[S+1] so that it holds vals [val_pos[i], val_pos[i+1]), used[S] = the
 * `first` flag of the slice (0 for an empty slice). keys/lens follow memkind;
 * lens == NULL or nlens == 0 means no lens (value length k = nvals / n).
 * `device` must be the device that holds PSKV_MEM_DEVICE inputs: those are searched (and their
 * lens added up per slice) by HIP kernels, one launch and one wait. PSKV_MEM_HOST inputs are
 * sliced where they lie, on the calling thread, with the reference's own loop: S+1 binary
 * searches touch a few dozen keys, and shipping n keys over the host link for them would cost
 * milliseconds at model size (this is by design, not a fallback: with PSKV_MEM_DEVICE inputs and
 * no GPU the call fails with PSKV_EHIP). */
int pskv_slice(int device, const uint64_t* keys, size_t n, const int32_t* lens, size_t nlens,
               size_t nvals, const uint64_t* range_begin, const uint64_t* range_end, size_t S,
               uint64_t* pos, uint64_t* val_pos, uint8_t* used, int memkind);

/* pskv_slice for callers that cannot allocate. It has no counterpart in the reference: it is
 * for code that may not call hipMalloc (under HIP graph capture, in tight serving loops, in
 * harnesses that forbid it). It allocates nothing and waits for nothing: the kernels are
 * enqueued on `stream` (a hipStream_t, NULL = the null stream) and their working memory (the
 * lower bounds of the searches and the per-slice sums of lens) is a fixed array inside the
 * library's code object, which every GPU that loads the library holds until the process ends
 * (about 16 KiB); that bounds S by PSKV_SLICE_NOALLOC_MAX_RANGES.
 * keys/lens are device memory on `device`; range_begin/range_end are host arrays, read before
 * the call returns; pos[S+1], val_pos[S+1], used[S] and status[1] are DEVICE memory, valid once
 * the stream has run the call. *status receives what pskv_slice would have returned for the
 * data-dependent outcomes (PSKV_OK, PSKV_EUNCOVERED_KEY, PSKV_ESIZE_MISMATCH); on a non-zero
 * status val_pos is unspecified. What the host can decide alone (null arguments, no range or
 * too many, a gap between ranges) is returned at once and nothing is enqueued.
 * All calls on one GPU share the one array: calls that overlap in time on a GPU (different
 * streams, or several threads) race; put them on one stream or order them with events.
 * The first call on a device looks the array's address up in the runtime: make it outside any
 * graph capture (a call with n = 0 will do). */
#define PSKV_SLICE_NOALLOC_MAX_RANGES 1024
int pskv_slice_noalloc(int device, void* stream, const uint64_t* keys, size_t n, const int32_t* lens,
                       size_t nlens, size_t nvals, const uint64_t* range_begin,
                       const uint64_t* range_end, size_t S, uint64_t* pos, uint64_t* val_pos,
                       uint8_t* used, int32_t* status);

/* Postoffice::GetServerKeyRanges (src/postoffice.cc:169-180) for num_servers
 * servers; host arrays of num_servers entries each. */
int pskv_server_ranges(uint64_t num_servers, uint64_t* range_begin, uint64_t* range_end);

/* Worker-side pull reassembly, the callback of KVWorker::AddPullCB
 * (kv_app.h:663-714): R per-server responses, in any order, are checked against
 * the request keys, ordered by first key and concatenated into out (and
 * out_lens when resp_lens is not NULL). The pointer tables and the size tables are
 * host arrays; what they point to follows memkind, as do req_keys/out/out_lens. */
int pskv_assemble_pull(int device, const uint64_t* req_keys, size_t n, size_t R,
                       const uint64_t* const* resp_keys, const size_t* resp_nkeys,
                       const float* const* resp_vals, const size_t* resp_nvals,
                       const int32_t* const* resp_lens, float* out, size_t out_cap,
                       int32_t* out_lens, size_t* out_nvals, int memkind);

/* Ordered match of two sorted key sets, ParallelOrderedMatch
 * (include/ps/internal/parallel_kv_match.h:29-120; operators: assign_op.h:12-41):
 *     if (dst_keys[i] == src_keys[j])  dst_vals[i*k .. i*k+k)  op=  src_vals[j*k .. j*k+k)
 * for sorted unique keys (a key set that repeats a key is a caller error with an unspecified
 * result, as the reference's "Keys must be unique and sorted", :79). Destination values without
 * a matching source key are left as they are. *matched (may be NULL) = k times the number of
 * matched keys: the reference counts values (:52). The bit operators of assign_op.h:20-22 are
 * for integers only (:38) and give PSKV_EINVAL here. The call returns when dst_vals is complete;
 * calls on one device take turns. kernel_ms (no counterpart in the reference) is NULL or room for
 * two floats: the device time of this call's key kernel and of its row kernel (0 for k == 1,
 * which needs none), read from events that the launches carry. */
#define PSKV_OP_ASSIGN 0 /* a = b */
#define PSKV_OP_PLUS 1   /* a += b */
#define PSKV_OP_MINUS 2  /* a -= b */
#define PSKV_OP_TIMES 3  /* a *= b */
#define PSKV_OP_DIVIDE 4 /* a /= b (assign_op.h:17 says "a -= b"; the code divides, :34) */
int pskv_match(int device, const uint64_t* src_keys, size_t n_src, const float* src_vals,
               const uint64_t* dst_keys, size_t n_dst, float* dst_vals, size_t k, int op,
               uint64_t* matched, float* kernel_ms, int memkind);

/* Device-time accounting for roofline figures (no counterpart in the reference).
 * While enabled, every launch of the kernels listed above is bracketed by HIP
 * events on the table's stream. pskv_prof_read waits for the stream and returns
 * the launch count and the summed duration since the last pskv_prof_reset. */
int pskv_prof_enable(pskv_table* t, int on);
int pskv_prof_reset(pskv_table* t);
int pskv_prof_read(pskv_table* t, int kernel, uint64_t* launches, double* total_ms);
/* The durations of the individual launches (in launch order) since the last
 * pskv_prof_reset, for medians and minima: writes min(*n, cap) values to out_ms and
 * the number recorded to *n. At most 65536 launches per kernel are kept. */
int pskv_prof_samples(pskv_table* t, int kernel, float* out_ms, size_t cap, size_t* n);

/* Plain device-to-device copy kernel of `bytes` bytes (multiple of 16) on the
 * table's stream; used to calibrate memory-traffic counters and as the measured
 * copy ceiling next to the accumulate kernels. No counterpart in the reference. */
int pskv_copy_probe(pskv_table* t, void* dst, const void* src, size_t bytes);

/* Pinned host memory for request/response buffers handed to PSKV_MEM_HOST calls
 * (copies to and from it run as DMA). pskv_host_free may be called from any thread
 * and never blocks in the GPU runtime: it only returns the buffer to a free list, as
 * a ps-lite response buffer is released on a transport thread
 * (src/zmq_van.h:20-26,159-175; SArray::reset with a deleter, sarray.h:162-165).
 * pskv_host_trim gives the free list back to the system. */
void* pskv_host_alloc(size_t bytes);
void pskv_host_free(void* ptr);
int pskv_host_trim(void);

/* What the sizing logic of a table has done so far (no counterpart in the reference; host-side
 * bookkeeping, no device work): writes min(cap, PSKV_COUNTER_COUNT) values to out, in this order. */
#define PSKV_COUNTER_REQUESTS 0        /* requests that could create keys */
#define PSKV_COUNTER_GROWTHS 1         /* times the slot array was replaced by a larger one */
#define PSKV_COUNTER_GROWTHS_UNASKED 2 /* ... decided from the host's bounds, without a wait */
#define PSKV_COUNTER_GROWTHS_AHEAD 3   /* ... into an array that had been allocated ahead of need */
#define PSKV_COUNTER_WAITS 4           /* waits for the stream to read exact counters */
#define PSKV_COUNTER_CATCH_UPS 5       /* times the host let the device catch up on published counters */
#define PSKV_COUNTER_RECORDS 6         /* requests that were asked to publish the counters */
#define PSKV_COUNTER_SLOTS 7           /* slots of the array now */
#define PSKV_COUNTER_COUNT 8
int pskv_table_counters(pskv_table* t, uint64_t* out, size_t cap);

/* Device memory the library keeps for reuse goes back to the system (no counterpart in the
 * reference): the slot arrays and row storage that growths have replaced (they stay in a
 * memory pool of the library, one per device, because releasing a few hundred MB costs
 * hundreds of microseconds that would land in the caller's next wait; the pool reuses them
 * for later growths of any table, and gives them up when this is called) and the workspaces
 * and staging buffers of pskv_match, which only grow (a 16M-key host-resident call leaves
 * several GiB behind). Memory in use by live tables is not touched. Calls of pskv_match on
 * the device wait for it and it for them. */
int pskv_device_trim(int device);

/* Text of the last error on the calling thread ("" if none). */
const char* pskv_last_error(void);
/* "pskv <major>.<minor> gfx950" */
const char* pskv_version(void);

#ifdef __cplusplus
}
#endif
#endif /* PSKV_CAPI_H_ */
