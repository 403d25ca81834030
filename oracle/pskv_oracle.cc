/*
 * CPU oracle: single-threaded restatement of ps-lite's slicer and default
 * request handle. TEST INFRASTRUCTURE ONLY (see pskv_oracle.h).
 *
 * The code deliberately stays close to the control flow of the reference so
 * that each CHECK of the reference maps to one early return here.
 */
#include "pskv_oracle.h"

#include <algorithm>
#include <cstring>
#include <limits>
#include <new>
#include <unordered_map>
#include <utility>
#include <vector>

namespace {

const uint64_t kMaxKey = std::numeric_limits<uint64_t>::max();  // include/ps/base.h:18
const uint64_t kMaxVarRow = (1ull << 28) - 1;                   // extended rule: var-len row limit

// Row of the extended stores. `len` is kept apart from data.size() only for clarity.
struct Row {
  std::vector<float> data;
};

}  // namespace

struct pskv_oracle_store {
  int mode;
  uint64_t row_len;                              // FIXED: floats per key (0 = unknown yet)
  std::unordered_map<uint64_t, float> scalar;    // kv_app.h:462
  std::unordered_map<uint64_t, Row> rows;        // extended stores
};

extern "C" {

// src/postoffice.cc:169-180
void pskv_oracle_server_ranges(uint64_t num_servers, uint64_t* begin, uint64_t* end) {
  for (uint64_t i = 0; i < num_servers; ++i) {
    begin[i] = kMaxKey / num_servers * i;
    end[i] = kMaxKey / num_servers * (i + 1);
  }
}

// include/ps/kv_app.h:517-572
int pskv_oracle_slice(const uint64_t* keys, size_t n_keys, const int32_t* lens, size_t nlens,
                      size_t nvals, const uint64_t* range_begin, const uint64_t* range_end,
                      size_t S, uint64_t* pos, uint64_t* val_pos, uint8_t* used) {
  // kv_app.h:524-541 : key positions
  const uint64_t* begin = keys;
  const uint64_t* end = keys + n_keys;
  for (size_t i = 0; i <= S; ++i) pos[i] = 0;
  for (size_t i = 0; i <= S; ++i) val_pos[i] = 0;
  for (size_t i = 0; i < S; ++i) {
    if (i == 0) {
      pos[0] = std::lower_bound(begin, end, range_begin[0]) - begin;  // :530
      begin += pos[0];
    } else if (range_end[i - 1] != range_begin[i]) {                  // :533
      return PSKV_ORACLE_ERANGE_GAP;
    }
    size_t len = std::lower_bound(begin, end, range_end[i]) - begin;  // :535
    begin += len;
    pos[i + 1] = pos[i] + len;
    used[i] = (len != 0);                                             // :540
  }
  if (pos[S] != n_keys) return PSKV_ORACLE_EUNCOVERED_KEY;            // :542
  if (n_keys == 0) return PSKV_ORACLE_OK;                             // :543

  // kv_app.h:546-552 : the length of a value
  size_t k = 0, val_begin = 0, val_end = 0;
  const bool has_lens = (lens != nullptr && nlens != 0);
  if (!has_lens) {
    k = nvals / n_keys;
    if (k * n_keys != nvals) return PSKV_ORACLE_ESIZE_MISMATCH;       // :549
  } else if (n_keys != nlens) {
    return PSKV_ORACLE_ESIZE_MISMATCH;                                // :551
  }

  // kv_app.h:555-571 : value offsets of every slice
  for (size_t i = 0; i < S; ++i) {
    if (pos[i + 1] == pos[i]) {
      used[i] = 0;
      val_pos[i + 1] = has_lens ? val_end : pos[i + 1] * k;
      continue;
    }
    used[i] = 1;
    if (has_lens) {
      // :565 `for (int l : kv.lens) val_end += l;` in size_t arithmetic
      for (size_t j = pos[i]; j < pos[i + 1]; ++j) val_end += static_cast<size_t>(lens[j]);
      // SArray::segment, sarray.h:249 : CHECK_GE(end, begin); CHECK_LE(end, size())
      if (val_end < val_begin || val_end > nvals) return PSKV_ORACLE_ESIZE_MISMATCH;
      val_pos[i] = val_begin;
      val_pos[i + 1] = val_end;
      val_begin = val_end;                                            // :567
    } else {
      val_pos[i] = pos[i] * k;                                        // :569
      val_pos[i + 1] = pos[i + 1] * k;
    }
  }
  if (!has_lens) {
    // slices are contiguous, so one running array describes all of them
    for (size_t i = 0; i <= S; ++i) val_pos[i] = pos[i] * k;
  }
  return PSKV_ORACLE_OK;
}

pskv_oracle_store* pskv_oracle_store_create(int mode, uint64_t row_len) {
  if (mode < PSKV_ORACLE_MODE_SCALAR || mode > PSKV_ORACLE_MODE_VARLEN) return nullptr;
  pskv_oracle_store* s = new (std::nothrow) pskv_oracle_store();
  if (!s) return nullptr;
  s->mode = mode;
  s->row_len = (mode == PSKV_ORACLE_MODE_SCALAR) ? 1 : row_len;
  return s;
}

void pskv_oracle_store_destroy(pskv_oracle_store* s) { delete s; }

size_t pskv_oracle_store_size(const pskv_oracle_store* s) {
  return s->mode == PSKV_ORACLE_MODE_SCALAR ? s->scalar.size() : s->rows.size();
}

size_t pskv_oracle_store_nvals(const pskv_oracle_store* s) {
  if (s->mode == PSKV_ORACLE_MODE_SCALAR) return s->scalar.size();
  size_t t = 0;
  for (const auto& kv : s->rows) t += kv.second.data.size();
  return t;
}

// Scalar store: KVServerDefaultHandle::operator(), include/ps/kv_app.h:442-461
static int handle_scalar(pskv_oracle_store* s, bool push, bool pull, const uint64_t* keys,
                         size_t n, const float* vals, size_t nvals, float* out_vals,
                         size_t out_cap, size_t* out_nvals) {
  if (!pull) {
    if (n != nvals) return PSKV_ORACLE_ESIZE_MISMATCH;  // :447
  } else if (push && n != nvals) {
    // The reference indexes vals[i] for i<n without a check here (:454); fewer
    // values would be an out-of-bounds read, so the oracle refuses the request.
    return PSKV_ORACLE_ESIZE_MISMATCH;
  }
  const bool can_write = pull && out_cap >= n;
  if (pull && out_nvals) *out_nvals = n;                // :449 res.vals.resize(n)
  for (size_t i = 0; i < n; ++i) {                      // :451
    uint64_t key = keys[i];
    if (push) s->scalar[key] += vals[i];                // :454 (absent key: 0.0f + v)
    if (pull) {
      float v = s->scalar[key];                         // :457 (absent key is inserted as 0)
      if (can_write) out_vals[i] = v;
    }
  }
  if (pull && !can_write) return PSKV_ORACLE_ESIZE_MISMATCH;
  return PSKV_ORACLE_OK;
}

// Extended store, fixed row length. Layout of vals: include/ps/kv_app.h:17-22.
static int handle_fixed(pskv_oracle_store* s, bool push, bool pull, const uint64_t* keys,
                        size_t n, const float* vals, size_t nvals, float* out_vals,
                        size_t out_cap, size_t* out_nvals) {
  if (push) {
    if (n == 0) {
      if (nvals != 0) return PSKV_ORACLE_ESIZE_MISMATCH;
    } else {
      uint64_t k = nvals / n;                                         // kv_app.h:548
      if (k * n != nvals || k == 0) return PSKV_ORACLE_ESIZE_MISMATCH;  // :549
      if (s->row_len == 0) s->row_len = k;
      if (k != s->row_len) return PSKV_ORACLE_ESIZE_MISMATCH;
    }
  }
  if (n == 0) {
    if (pull && out_nvals) *out_nvals = 0;
    return PSKV_ORACLE_OK;
  }
  const uint64_t k = s->row_len;
  if (k == 0) return PSKV_ORACLE_EINVAL;  // pull before the row length is known
  const bool can_write = pull && out_cap >= n * k;
  if (pull && out_nvals) *out_nvals = n * k;
  for (size_t i = 0; i < n; ++i) {
    Row& r = s->rows[keys[i]];
    if (r.data.empty()) r.data.assign(k, 0.0f);  // first touch: a zero row
    if (push) {
      const float* in = vals + i * k;
      for (uint64_t j = 0; j < k; ++j) r.data[j] += in[j];
    }
    if (pull && can_write) std::memcpy(out_vals + i * k, r.data.data(), k * sizeof(float));
  }
  if (pull && !can_write) return PSKV_ORACLE_ESIZE_MISMATCH;
  return PSKV_ORACLE_OK;
}

// Extended store, per-key row length. Layout of vals/lens: include/ps/kv_app.h:24-31.
static int handle_varlen(pskv_oracle_store* s, bool push, bool pull, const uint64_t* keys,
                         size_t n, const float* vals, size_t nvals, const int32_t* lens,
                         size_t nlens, float* out_vals, size_t out_cap, int32_t* out_lens,
                         size_t* out_nvals) {
  if (push) {
    if (nlens != n) return PSKV_ORACLE_ESIZE_MISMATCH;  // kv_app.h:489,551
    uint64_t total = 0;
    for (size_t i = 0; i < n; ++i) {
      if (lens[i] < 0 || static_cast<uint64_t>(lens[i]) > kMaxVarRow) return PSKV_ORACLE_EINVAL;
      total += static_cast<uint64_t>(lens[i]);
    }
    if (total != nvals) return PSKV_ORACLE_ESIZE_MISMATCH;
    // A row never changes its length. Absent keys are created (as zero rows)
    // before the decision, present rows are only touched when every length matches.
    bool changed = false;
    for (size_t i = 0; i < n; ++i) {
      auto it = s->rows.find(keys[i]);
      if (it == s->rows.end()) {
        s->rows[keys[i]].data.assign(static_cast<size_t>(lens[i]), 0.0f);
      } else if (it->second.data.size() != static_cast<size_t>(lens[i])) {
        changed = true;
      }
    }
    if (changed) return PSKV_ORACLE_ELEN_CHANGED;
    size_t off = 0;
    for (size_t i = 0; i < n; ++i) {
      Row& r = s->rows[keys[i]];
      for (size_t j = 0; j < r.data.size(); ++j) r.data[j] += vals[off + j];
      off += r.data.size();
    }
  }
  if (pull) {
    size_t total = 0;
    for (size_t i = 0; i < n; ++i) {
      auto it = s->rows.find(keys[i]);  // an absent key answers len 0 and is not created
      size_t l = (it == s->rows.end()) ? 0 : it->second.data.size();
      if (out_lens) out_lens[i] = static_cast<int32_t>(l);
      total += l;
    }
    if (out_nvals) *out_nvals = total;
    if (total > out_cap) return PSKV_ORACLE_ESIZE_MISMATCH;
    size_t off = 0;
    for (size_t i = 0; i < n; ++i) {
      auto it = s->rows.find(keys[i]);
      if (it == s->rows.end()) continue;
      const std::vector<float>& d = it->second.data;
      if (!d.empty()) std::memcpy(out_vals + off, d.data(), d.size() * sizeof(float));
      off += d.size();
    }
  }
  return PSKV_ORACLE_OK;
}

int pskv_oracle_handle(pskv_oracle_store* s, int push, int pull, const uint64_t* keys, size_t n,
                       const float* vals, size_t nvals, const int32_t* lens, size_t nlens,
                       float* out_vals, size_t out_cap, int32_t* out_lens, size_t* out_nvals) {
  if (!s) return PSKV_ORACLE_EINVAL;
  if (out_nvals) *out_nvals = 0;
  try {
    switch (s->mode) {
      case PSKV_ORACLE_MODE_SCALAR:
        return handle_scalar(s, push != 0, pull != 0, keys, n, vals, nvals, out_vals, out_cap,
                             out_nvals);
      case PSKV_ORACLE_MODE_FIXED:
        return handle_fixed(s, push != 0, pull != 0, keys, n, vals, nvals, out_vals, out_cap,
                            out_nvals);
      default:
        return handle_varlen(s, push != 0, pull != 0, keys, n, vals, nvals, lens, nlens,
                             out_vals, out_cap, out_lens, out_nvals);
    }
  } catch (const std::bad_alloc&) {
    return PSKV_ORACLE_ENOMEM;
  }
}

int pskv_oracle_store_dump(const pskv_oracle_store* s, uint64_t* keys, int32_t* lens,
                           size_t cap_keys, float* vals, size_t cap_vals, size_t* n_keys,
                           size_t* n_vals) {
  const size_t nk = pskv_oracle_store_size(s);
  const size_t nv = pskv_oracle_store_nvals(s);
  if (n_keys) *n_keys = nk;
  if (n_vals) *n_vals = nv;
  if (nk > cap_keys || nv > cap_vals) return PSKV_ORACLE_ESIZE_MISMATCH;
  std::vector<uint64_t> order;
  order.reserve(nk);
  if (s->mode == PSKV_ORACLE_MODE_SCALAR) {
    for (const auto& kv : s->scalar) order.push_back(kv.first);
  } else {
    for (const auto& kv : s->rows) order.push_back(kv.first);
  }
  std::sort(order.begin(), order.end());
  size_t off = 0;
  for (size_t i = 0; i < nk; ++i) {
    keys[i] = order[i];
    if (s->mode == PSKV_ORACLE_MODE_SCALAR) {
      vals[off++] = s->scalar.find(order[i])->second;
      if (lens) lens[i] = 1;
    } else {
      const std::vector<float>& d = s->rows.find(order[i])->second.data;
      if (!d.empty()) std::memcpy(vals + off, d.data(), d.size() * sizeof(float));
      off += d.size();
      if (lens) lens[i] = static_cast<int32_t>(d.size());
    }
  }
  return PSKV_ORACLE_OK;
}

// include/ps/sarray.h:281-287
void pskv_oracle_find_range(const uint64_t* arr, size_t n, uint64_t lower, uint64_t upper,
                            uint64_t* begin, uint64_t* end) {
  if (upper <= lower) {
    *begin = 0;
    *end = 0;
    return;
  }
  *begin = std::lower_bound(arr, arr + n, lower) - arr;
  *end = std::lower_bound(arr, arr + n, upper) - arr;
}

// include/ps/kv_app.h:663-714
int pskv_oracle_assemble_pull(const uint64_t* req_keys, size_t n, size_t R,
                              const uint64_t* const* resp_keys, const size_t* resp_nkeys,
                              const float* const* resp_vals, const size_t* resp_nvals,
                              const int32_t* const* resp_lens, float* out_vals, size_t out_cap,
                              int32_t* out_lens, size_t* out_nvals) {
  size_t total_key = 0, total_val = 0;
  for (size_t r = 0; r < R; ++r) {  // :670-677
    if (resp_nkeys[r] == 0) return PSKV_ORACLE_EINVAL;  // front()/back() CHECK(!empty())
    uint64_t b, e;
    // back()+1 wraps to 0 for kMaxKey exactly as the reference's Key arithmetic does
    pskv_oracle_find_range(req_keys, n, resp_keys[r][0], resp_keys[r][resp_nkeys[r] - 1] + 1, &b,
                           &e);
    if (e - b != resp_nkeys[r]) return PSKV_ORACLE_ESIZE_MISMATCH;  // :672
    total_key += resp_nkeys[r];
    total_val += resp_nvals[r];
  }
  if (total_key != n) return PSKV_ORACLE_ESIZE_MISMATCH;  // :678
  std::vector<size_t> order(R);
  for (size_t r = 0; r < R; ++r) order[r] = r;
  std::sort(order.begin(), order.end(), [&](size_t a, size_t b) {  // :681-684
    return resp_keys[a][0] < resp_keys[b][0];
  });
  if (out_nvals) *out_nvals = total_val;
  if (total_val > out_cap) return PSKV_ORACLE_ESIZE_MISMATCH;  // :686-690
  size_t voff = 0, koff = 0;
  for (size_t i = 0; i < R; ++i) {  // :701-708
    size_t r = order[i];
    if (resp_nvals[r]) std::memcpy(out_vals + voff, resp_vals[r], resp_nvals[r] * sizeof(float));
    voff += resp_nvals[r];
    if (out_lens && resp_lens) {
      std::memcpy(out_lens + koff, resp_lens[r], resp_nkeys[r] * sizeof(int32_t));
    }
    koff += resp_nkeys[r];
  }
  return PSKV_ORACLE_OK;
}

// include/ps/internal/parallel_kv_match.h:29-60 with the operators of assign_op.h:12-41. The
// reference splits dst in halves over threads (:61-73); every half runs the loop below on its
// own dst range against the whole of src, so the sequential loop gives the same result.
int pskv_oracle_ordered_match(const uint64_t* src_keys, size_t n_src, const float* src_vals,
                              const uint64_t* dst_keys, size_t n_dst, float* dst_vals, size_t k,
                              int op, size_t* matched) {
  if (matched) *matched = 0;
  if (op < 0 || op > 4) return PSKV_ORACLE_EINVAL;  // assign_op.h:38: the bit operators are for integers
  if (n_dst == 0 || n_src == 0) return PSKV_ORACLE_OK;  // :36
  const uint64_t* src_end = src_keys + n_src;
  const uint64_t* dst_end = dst_keys + n_dst;
  const uint64_t* sk = std::lower_bound(src_keys, src_end, *dst_keys);  // :39
  const float* sv = src_vals + (sk - src_keys) * k;                     // :40
  const uint64_t* dk = dst_keys;
  float* dv = dst_vals;
  size_t n = 0;
  while (dk != dst_end && sk != src_end) {  // :43-58
    if (*sk < *dk) {
      ++sk;
      sv += k;
    } else {
      if (!(*dk < *sk)) {
        for (size_t i = 0; i < k; ++i) {
          switch (op) {  // assign_op.h:26-36: right op= left
            case 0: dv[i] = sv[i]; break;
            case 1: dv[i] += sv[i]; break;
            case 2: dv[i] -= sv[i]; break;
            case 3: dv[i] *= sv[i]; break;
            case 4: dv[i] /= sv[i]; break;
          }
        }
        ++sk;
        sv += k;
        n += k;  // :52 counts values, not keys
      }
      ++dk;
      dv += k;
    }
  }
  if (matched) *matched = n;
  return PSKV_ORACLE_OK;
}

}  // extern "C"
