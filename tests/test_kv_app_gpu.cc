// The reference's key-value integration test (tests/test_kv_app.cc) run against the GPU
// slicer and the GPU request handle through the in-process ps:: surface: the same
// worker program, the same closed forms, plus the multi-float layouts and the failure
// cases of the data path, and the two-workers-in-one-process variant
// (tests/test_kv_app_multi_workers.cc).
//
//   test_kv_app_gpu [num_servers [floats per key of the dense run from host memory]]
#include <atomic>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <memory>
#include <string>
#include <thread>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "pskv/ps_min.h"
#include "pskv/ps_adapters.h"

using namespace ps;

static std::atomic<int> g_failures(0);
#define EXPECT(cond)                                                        \
  do {                                                                      \
    if (!(cond)) {                                                          \
      std::fprintf(stderr, "%s:%d: EXPECT failed: %s\n", __FILE__, __LINE__, #cond); \
      ++g_failures;                                                         \
    }                                                                       \
  } while (0)

static std::vector<std::unique_ptr<KVServer<float>>> StartServers(int app_id, int num, int mode) {
  std::vector<std::unique_ptr<KVServer<float>>> servers;
  for (int i = 0; i < num; ++i) {
    servers.emplace_back(new KVServer<float>(app_id));
    pskv_opts o = pskv_opts();
    o.mode = mode;
    o.initial_capacity = 1024;
    servers.back()->set_request_handle(pskv::GpuKVHandle<float>(o));  // tests/test_kv_app.cc:10-11
  }
  return servers;
}

// tests/test_kv_app.cc:15-62
static void RunWorker(int app_id, int num, bool ones) {
  KVWorker<float> kv(app_id, 0);
  kv.set_slicer(pskv::GpuSlicer<float>(0));
  std::vector<Key> keys(num);
  std::vector<float> vals(num);
  const int rank = 0;
  srand(rank + 7);
  for (int i = 0; i < num; ++i) {
    keys[i] = kMaxKey / num * i + rank;
    vals[i] = ones ? 1.0f : static_cast<float>(rand() % 1000);
  }
  const int repeat = 50;
  std::vector<int> ts;
  {
    // untimed: the first request through a fresh process loads the GPU code and creates the
    // slicer's context; pushing zeros leaves every sum as it is
    std::vector<float> zeros(num, 0.0f), tmp;
    kv.Wait(kv.Push(keys, zeros));
    kv.Wait(kv.Pull(keys, &tmp));
  }
  const auto t_begin = std::chrono::steady_clock::now();
  for (int i = 0; i < repeat; ++i) {
    ts.push_back(kv.Push(keys, vals));
    if (i > 10) kv.Wait(ts[ts.size() - 10]);
  }
  for (int t : ts) kv.Wait(t);

  std::vector<float> rets;
  kv.Wait(kv.Pull(keys, &rets));
  const double push_pull_ms =
      std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t_begin).count();

  std::vector<float> outs;
  for (int i = 0; i < repeat; ++i) kv.Wait(kv.PushPull(keys, vals, &outs));

  float res = 0, res2 = 0;
  for (int i = 0; i < num; ++i) {
    res += std::fabs(rets[i] - vals[i] * repeat);
    res2 += std::fabs(outs[i] - vals[i] * 2 * repeat);
  }
  EXPECT(rets.size() == static_cast<size_t>(num));
  EXPECT(res / repeat < 1e-5);
  EXPECT(res2 / (2 * repeat) < 1e-5);
  // integer-valued floats below 2^24 add exactly, so the sums are not merely close
  EXPECT(res == 0.0f && res2 == 0.0f);
  std::printf("kv_app num=%d error: %g, %g; %d pushes + 1 pull through slicer, handle and host staging: %.2f ms\n",
              num, res / repeat, res2 / (2 * repeat), repeat, push_pull_ms);
}

// tests/test_kv_app_multi_workers.cc:12-60: one of two workers of a process, each on a thread of
// its own with its own customer id; the key sets interleave (keys offset by the customer id), so
// every server sees requests of both workers in whatever order the threads get there, and every
// GpuSlicer call may run next to the other worker's.
static void RunOneOfTwoWorkers(int app_id, int customer_id) {
  try {
    KVWorker<float> kv(app_id, customer_id);
    kv.set_slicer(pskv::GpuSlicer<float>(0));
    const int num = 10000;
    std::vector<Key> keys(num);
    std::vector<float> vals(num);
    unsigned seed = 7u + static_cast<unsigned>(customer_id);
    for (int i = 0; i < num; ++i) {
      keys[i] = kMaxKey / num * i + customer_id;
      seed = seed * 1103515245u + 12345u;
      vals[i] = static_cast<float>((seed >> 16) % 1000);
    }
    const int repeat = 50;
    std::vector<int> ts;
    for (int i = 0; i < repeat; ++i) {
      ts.push_back(kv.Push(keys, vals));
      if (i > 10) kv.Wait(ts[ts.size() - 10]);
    }
    for (int t : ts) kv.Wait(t);
    std::vector<float> rets;
    kv.Wait(kv.Pull(keys, &rets));
    std::vector<float> outs;
    for (int i = 0; i < repeat; ++i) kv.Wait(kv.PushPull(keys, vals, &outs));
    float res = 0, res2 = 0;
    for (int i = 0; i < num; ++i) {
      res += std::fabs(rets[i] - vals[i] * repeat);
      res2 += std::fabs(outs[i] - vals[i] * 2 * repeat);  // (the reference never adds to res2, :53-57)
    }
    EXPECT(rets.size() == static_cast<size_t>(num) && outs.size() == static_cast<size_t>(num));
    EXPECT(res == 0.0f && res2 == 0.0f);
    std::printf("kv_app two workers, customer %d: error %g, %g\n", customer_id, res / repeat, res2 / (2 * repeat));
  } catch (const std::exception& e) {
    std::fprintf(stderr, "worker %d: unexpected exception: %s\n", customer_id, e.what());
    ++g_failures;
  }
}

// The merge a worker does with what it pulled (parallel_kv_match.h:76-94): values of the keys
// that both sides hold are combined, the others stay; a destination that is too short grows
// with zeros first.
static void RunOrderedMatch() {
  const int num = 5000, k = 2;
  SArray<Key> src_key(num), dst_key(num);
  SArray<float> src_val(num * k);
  for (int i = 0; i < num; ++i) {
    src_key[i] = static_cast<Key>(3 * i);      // multiples of 3
    dst_key[i] = static_cast<Key>(2 * i + 6);  // even numbers from 6: every third one matches
    src_val[2 * i] = static_cast<float>(i);
    src_val[2 * i + 1] = static_cast<float>(-i);
  }
  std::vector<float> dst_val(10, 100.0f);  // the first five keys hold 100, the rest come as 0
  const size_t n = pskv::GpuOrderedMatch(src_key, src_val, dst_key, &dst_val, k, PSKV_OP_PLUS);
  size_t want_n = 0;
  bool ok = dst_val.size() == static_cast<size_t>(num) * k;
  for (int i = 0; i < num && ok; ++i) {
    const Key key = dst_key[i];
    float a = i < 5 ? 100.0f : 0.0f, b = a;
    if (key % 3 == 0 && key / 3 < static_cast<Key>(num)) {
      a += static_cast<float>(key / 3);
      b -= static_cast<float>(key / 3);
      want_n += k;
    }
    ok = dst_val[2 * i] == a && dst_val[2 * i + 1] == b;
  }
  EXPECT(ok);
  EXPECT(n == want_n);
  bool threw = false;
  try {
    pskv::GpuOrderedMatch(src_key, src_val, dst_key, &dst_val, 3, PSKV_OP_PLUS);  // 3 values per key: sizes do not fit
  } catch (const dmlc::Error&) {
    threw = true;
  }
  EXPECT(threw);
  std::printf("ordered match: %zu of %d values matched\n", n, num * k);
}

// The contract of device-resident calls, through the C ABI alone (nothing keeps the buffers alive
// for the caller here): a PSKV_MEM_DEVICE call only enqueues work; the table reads the request's
// buffers, and writes the response, some time before the next pskv_sync returns; after that wait
// the buffers are the caller's again and may be overwritten or freed. 150,000 keys, above the size
// from which SCALAR tables keep a request-ordered copy of the last key set, so the pushes also go
// through that copy; every push brings other values in the SAME device buffer.
static void RunDeviceBufferContract() {
  const size_t n = 150000;
  const int pushes = 12;
  pskv_opts o = {};
  o.mode = PSKV_MODE_SCALAR;
  pskv_table* t = nullptr;
  EXPECT(pskv_table_create(&t, &o) == PSKV_OK);
  std::vector<uint64_t> keys(n);
  std::vector<float> vals(n), want(n, 0.0f), got(n, -1.0f);
  for (size_t i = 0; i < n; ++i) keys[i] = (~0ull / n) * i + 17;
  uint64_t* d_keys = nullptr;
  float *d_vals = nullptr, *d_out = nullptr;
  EXPECT(hipMalloc(reinterpret_cast<void**>(&d_keys), n * 8) == hipSuccess);
  EXPECT(hipMalloc(reinterpret_cast<void**>(&d_vals), n * 4) == hipSuccess);
  EXPECT(hipMalloc(reinterpret_cast<void**>(&d_out), n * 4) == hipSuccess);
  EXPECT(hipMemcpy(d_keys, keys.data(), n * 8, hipMemcpyHostToDevice) == hipSuccess);
  for (int p = 0; p < pushes; ++p) {
    for (size_t i = 0; i < n; ++i) {
      vals[i] = static_cast<float>((i * 7 + p * 13) % 101) * 0.25f - 3.0f;
      want[i] = want[i] + vals[i];
    }
    // the buffer is the caller's here: the previous push has been waited for
    EXPECT(hipMemcpy(d_vals, vals.data(), n * 4, hipMemcpyHostToDevice) == hipSuccess);
    EXPECT(pskv_push(t, d_keys, n, d_vals, n, nullptr, 0, PSKV_MEM_DEVICE) == PSKV_OK);
    if (p % 3 == 1) EXPECT(pskv_pull(t, d_keys, n, d_out, n, nullptr, nullptr, PSKV_MEM_DEVICE) == PSKV_OK);
    EXPECT(pskv_sync(t) == PSKV_OK);  // from here on d_vals may change again
  }
  EXPECT(pskv_pull(t, d_keys, n, d_out, n, nullptr, nullptr, PSKV_MEM_DEVICE) == PSKV_OK);
  EXPECT(pskv_sync(t) == PSKV_OK);  // from here on d_out holds the response
  EXPECT(hipMemcpy(got.data(), d_out, n * 4, hipMemcpyDeviceToHost) == hipSuccess);
  size_t bad = 0;
  for (size_t i = 0; i < n; ++i) bad += got[i] != want[i];
  EXPECT(bad == 0);
  // buffers may be freed once the wait has returned, with the table still alive
  EXPECT(hipFree(d_vals) == hipSuccess);
  EXPECT(hipFree(d_out) == hipSuccess);
  EXPECT(hipFree(d_keys) == hipSuccess);
  uint64_t held = 0;
  EXPECT(pskv_size(t, &held, nullptr) == PSKV_OK && held == n);
  EXPECT(pskv_table_destroy(t) == PSKV_OK);
  std::printf("device buffers: %d pushes of %zu keys from one buffer, %zu floats differ\n", pushes, n, bad);
}

// The reference's test pushes one key set `repeat` times and pulls it once (tests/test_kv_app.cc:36-60).
// Here with the servers' tables and the worker's buffers on one GPU: the request is recorded once
// (pskv_replay_record) and every repeat is one pskv_replay_run; closed forms as in the reference's check.
static void RunRecordedRequests(int num_servers) {
  const size_t S = static_cast<size_t>(num_servers), n = 200000;
  const int repeat = 50;
  std::vector<uint64_t> rb(S), re(S), pos(S + 1), val_pos(S + 1);
  std::vector<uint8_t> used(S);
  EXPECT(pskv_server_ranges(S, rb.data(), re.data()) == PSKV_OK);
  std::vector<pskv_table*> t(S, nullptr);
  pskv_opts o = {};
  o.mode = PSKV_MODE_SCALAR;
  for (size_t s = 0; s < S; ++s) {
    EXPECT(pskv_table_create(&t[s], &o) == PSKV_OK);
    o.stream = pskv_table_stream(t[0]);
  }
  std::vector<uint64_t> keys(n);
  std::vector<float> vals(n), got(n, -1.0f);
  for (size_t i = 0; i < n; ++i) {
    keys[i] = (re[S - 1] / n) * i;  // tests/test_kv_app.cc:27
    vals[i] = static_cast<float>(i % 1000) * 0.5f;
  }
  uint64_t* d_keys = nullptr;
  float *d_vals = nullptr, *d_out = nullptr;
  EXPECT(hipMalloc(reinterpret_cast<void**>(&d_keys), n * 8) == hipSuccess);
  EXPECT(hipMalloc(reinterpret_cast<void**>(&d_vals), n * 4) == hipSuccess);
  EXPECT(hipMalloc(reinterpret_cast<void**>(&d_out), n * 4) == hipSuccess);
  EXPECT(hipMemcpy(d_keys, keys.data(), n * 8, hipMemcpyHostToDevice) == hipSuccess);
  EXPECT(hipMemcpy(d_vals, vals.data(), n * 4, hipMemcpyHostToDevice) == hipSuccess);
  EXPECT(pskv_slice(0, d_keys, n, nullptr, 0, n, rb.data(), re.data(), S, pos.data(), val_pos.data(), used.data(),
                    PSKV_MEM_DEVICE) == PSKV_OK);
  pskv_replay* push = nullptr;
  EXPECT(pskv_replay_record(&push, t.data(), S, PSKV_REPLAY_PUSH, d_keys, pos.data(), d_vals, val_pos.data(), nullptr,
                            nullptr, nullptr, nullptr) == PSKV_OK);  // push 1 of `repeat`
  for (int r = 1; r < repeat; ++r) EXPECT(pskv_replay_run(push) == PSKV_OK);
  EXPECT(pskv_pull_multi(t.data(), S, d_keys, pos.data(), d_out, nullptr, nullptr, nullptr, PSKV_MEM_DEVICE) == PSKV_OK);
  EXPECT(pskv_sync_multi(t.data(), S) == PSKV_OK);
  // the pull was another request: the recording is over
  EXPECT(pskv_replay_run(push) == PSKV_ESTALE);
  EXPECT(pskv_replay_destroy(push) == PSKV_OK);
  EXPECT(hipMemcpy(got.data(), d_out, n * 4, hipMemcpyDeviceToHost) == hipSuccess);
  size_t bad = 0;
  for (size_t i = 0; i < n; ++i) {
    float want = 0.0f;
    for (int r = 0; r < repeat; ++r) want = want + vals[i];  // sequential float adds, as the store makes them
    bad += got[i] != want;
  }
  EXPECT(bad == 0);
  // push + pull recorded as one step; a key that changes under the recording stops its slice, and only that
  pskv_replay* step = nullptr;
  EXPECT(pskv_replay_record(&step, t.data(), S, PSKV_REPLAY_PUSH | PSKV_REPLAY_PULL, d_keys, pos.data(), d_vals,
                            val_pos.data(), nullptr, d_out, nullptr, nullptr) == PSKV_OK);
  EXPECT(pskv_replay_run(step) == PSKV_OK);
  EXPECT(pskv_sync_multi(t.data(), S) == PSKV_OK);
  EXPECT(hipMemcpy(got.data(), d_out, n * 4, hipMemcpyDeviceToHost) == hipSuccess);
  size_t bad2 = 0;
  for (size_t i = 0; i < n; ++i) {
    float want = 0.0f;
    for (int r = 0; r < repeat + 2; ++r) want = want + vals[i];
    bad2 += got[i] != want;
  }
  EXPECT(bad2 == 0);
  const uint64_t other = keys[n - 1] + 1;  // the last key of the last slice becomes another key of its range
  EXPECT(hipMemcpy(d_keys + (n - 1), &other, 8, hipMemcpyHostToDevice) == hipSuccess);
  EXPECT(pskv_replay_run(step) == PSKV_OK);  // enqueued; the device finds the difference
  EXPECT(pskv_sync_multi(t.data(), S) == PSKV_ESTALE);
  uint64_t held = 0, total = 0;
  for (size_t s = 0; s < S; ++s) {
    EXPECT(pskv_size(t[s], &held, nullptr) == PSKV_OK);
    total += held;
  }
  EXPECT(total == n);  // the other key was not created
  EXPECT(pskv_replay_destroy(step) == PSKV_OK);
  EXPECT(hipFree(d_vals) == hipSuccess);
  EXPECT(hipFree(d_out) == hipSuccess);
  EXPECT(hipFree(d_keys) == hipSuccess);
  for (size_t s = S; s-- > 0;) EXPECT(pskv_table_destroy(t[s]) == PSKV_OK);  // the owner of the stream last
  std::printf("recorded requests: %d pushes of %zu keys over %zu ranges replayed, %zu + %zu floats differ\n", repeat, n,
              S, bad, bad2);
}

static void RunTwoWorkers(int app_id) {
  std::thread t0(RunOneOfTwoWorkers, app_id, 0);
  std::thread t1(RunOneOfTwoWorkers, app_id, 1);
  t0.join();
  t1.join();
}

// The example of kv_app.h:89-96: two keys with length-2 values.
static void RunFixed() {
  KVWorker<float> kv(1, 0);
  kv.set_slicer(pskv::GpuSlicer<float>(0));
  std::vector<Key> keys = {1, 3};
  std::vector<float> vals = {1.1f, 1.2f, 3.1f, 3.2f};
  kv.Wait(kv.Push(keys, vals));
  kv.Wait(kv.Push(keys, vals));
  std::vector<float> out;
  kv.Wait(kv.Pull(keys, &out));
  EXPECT(out.size() == 4);
  for (size_t i = 0; i < out.size() && i < 4; ++i) EXPECT(out[i] == (0.0f + vals[i]) + vals[i]);
  // keys spread over all servers, 3 floats each
  const int num = 999;
  std::vector<Key> k2(num);
  std::vector<float> v2(num * 4);
  for (int i = 0; i < num; ++i) k2[i] = kMaxKey / num * i + 5;
  for (size_t i = 0; i < v2.size(); ++i) v2[i] = static_cast<float>(i % 17) - 8.0f;
  KVWorker<float> kv2(2, 0);
  kv2.set_slicer(pskv::GpuSlicer<float>(0));
  for (int r = 0; r < 3; ++r) kv2.Wait(kv2.Push(k2, v2));
  std::vector<float> o2;
  kv2.Wait(kv2.Pull(k2, &o2));
  EXPECT(o2.size() == v2.size());
  for (size_t i = 0; i < o2.size() && i < v2.size(); ++i) EXPECT(o2[i] == 3 * v2[i]);
}

// Values of different lengths with lens (KVPairs layout, kv_app.h:24-31).
static void RunVarLen() {
  KVWorker<float> kv(3, 0);
  kv.set_slicer(pskv::GpuSlicer<float>(0));
  const int num = 2000;
  const int choices[5] = {8, 16, 32, 64, 128};
  std::vector<Key> keys(num);
  std::vector<int> lens(num);
  size_t total = 0;
  for (int i = 0; i < num; ++i) {
    keys[i] = kMaxKey / num * i + 11;
    lens[i] = choices[(i * 7) % 5];
    total += lens[i];
  }
  std::vector<float> vals(total);
  for (size_t i = 0; i < total; ++i) vals[i] = static_cast<float>(i % 29) - 14.0f;
  for (int r = 0; r < 4; ++r) kv.Wait(kv.Push(keys, vals, lens));
  std::vector<float> out;
  std::vector<int> out_lens;
  kv.Wait(kv.Pull(keys, &out, &out_lens));
  EXPECT(out.size() == total);
  EXPECT(out_lens == lens);
  for (size_t i = 0; i < out.size() && i < total; ++i) EXPECT(out[i] == 4 * vals[i]);
  // push and pull in one request: the push is applied once, then read back (kv_app.h:453-458)
  std::vector<float> both;
  std::vector<int> both_lens = lens;
  kv.Wait(kv.PushPull(keys, vals, &both, &both_lens));
  EXPECT(both.size() == total);
  EXPECT(both_lens == lens);
  for (size_t i = 0; i < both.size() && i < total; ++i) EXPECT(both[i] == 5 * vals[i]);
  // a small pull, then a larger one again: the handle sizes its response buffer from the last
  // response and must ask a second time when that guess is too small
  std::vector<Key> few(keys.begin(), keys.begin() + 10);
  std::vector<float> few_out;
  std::vector<int> few_lens;
  kv.Wait(kv.Pull(few, &few_out, &few_lens));
  size_t few_total = 0;
  for (int i = 0; i < 10; ++i) few_total += lens[i];
  EXPECT(few_out.size() == few_total);
  for (size_t i = 0; i < few_out.size() && i < few_total; ++i) EXPECT(few_out[i] == 5 * vals[i]);
  std::vector<float> again;
  std::vector<int> again_lens;
  kv.Wait(kv.Pull(keys, &again, &again_lens));
  EXPECT(again.size() == total);
  EXPECT(again_lens == lens);
  for (size_t i = 0; i < again.size() && i < total; ++i) EXPECT(again[i] == 5 * vals[i]);
}

// Dense chunks the way a ps-lite server gets them (BASELINE configuration 3: 64 keys of 4,194,304
// floats, 1 GiB per push): requests in ordinary host memory through the slicer and the request
// handle, the response in pinned buffers that the worker copies out of (kv_app.h:701-708). Prints
// the PCIe-inclusive rates; the sums are checked against their closed form.
static void RunDenseFromHost(size_t floats_per_key) {
  const int num = 64;
  KVWorker<float> kv(5, 0);
  kv.set_slicer(pskv::GpuSlicer<float>(0));
  std::vector<Key> keys(num);
  for (int i = 0; i < num; ++i) keys[i] = kMaxKey / num * i;
  std::vector<float> vals(num * floats_per_key);
  for (size_t i = 0; i < vals.size(); ++i) vals[i] = static_cast<float>(static_cast<int>(i % 251) - 125);
  const double gib = vals.size() * sizeof(float) / 1073741824.0;
  // the zero-copy calls (kv_app.h:243-258): Push/Pull would first copy the gigabyte into an SArray
  SArray<Key> zkeys(keys);
  SArray<float> zvals(vals);
  SArray<float> out(vals.size());
  kv.Wait(kv.ZPush(zkeys, zvals));  // creates the rows, warms the staging buffers up
  double best_push = 1e30, best_pull = 1e30;
  for (int r = 0; r < 3; ++r) {
    auto t0 = std::chrono::steady_clock::now();
    kv.Wait(kv.ZPush(zkeys, zvals));
    auto t1 = std::chrono::steady_clock::now();
    kv.Wait(kv.ZPull(zkeys, &out));
    auto t2 = std::chrono::steady_clock::now();
    best_push = std::min(best_push, std::chrono::duration<double>(t1 - t0).count());
    best_pull = std::min(best_pull, std::chrono::duration<double>(t2 - t1).count());
  }
  EXPECT(out.size() == vals.size());
  size_t bad = 0;
  for (size_t i = 0; i < out.size() && i < vals.size(); ++i) bad += out[i] != 4 * vals[i];
  EXPECT(bad == 0);
  std::printf("dense from host memory, %.2f GiB per request through GpuSlicer + GpuKVHandle: push %.1f GB/s, "
              "pull %.1f GB/s (the pull includes the worker's own copy out of the response)\n",
              gib, gib * 1.073741824 / best_push, gib * 1.073741824 / best_pull);
  // the C ABI alone, ordinary (pageable) buffers both ways
  pskv_opts o = pskv_opts();
  o.mode = PSKV_MODE_FIXED;
  o.row_len = floats_per_key;
  pskv_table* t = nullptr;
  EXPECT(pskv_table_create(&t, &o) == PSKV_OK);
  std::vector<uint64_t> k64(keys.begin(), keys.end());
  std::vector<float> out2(vals.size());
  EXPECT(pskv_push(t, k64.data(), num, vals.data(), vals.size(), nullptr, 0, PSKV_MEM_HOST) == PSKV_OK);
  best_push = best_pull = 1e30;
  size_t got = 0;
  for (int r = 0; r < 3; ++r) {
    auto t0 = std::chrono::steady_clock::now();
    EXPECT(pskv_push(t, k64.data(), num, vals.data(), vals.size(), nullptr, 0, PSKV_MEM_HOST) == PSKV_OK);
    auto t1 = std::chrono::steady_clock::now();
    EXPECT(pskv_pull(t, k64.data(), num, out2.data(), out2.size(), nullptr, &got, PSKV_MEM_HOST) == PSKV_OK);
    auto t2 = std::chrono::steady_clock::now();
    best_push = std::min(best_push, std::chrono::duration<double>(t1 - t0).count());
    best_pull = std::min(best_pull, std::chrono::duration<double>(t2 - t1).count());
  }
  bad = 0;
  for (size_t i = 0; i < out2.size(); ++i) bad += out2[i] != 4 * vals[i];
  EXPECT(bad == 0 && got == vals.size());
  std::printf("dense from host memory, %.2f GiB per request through pskv_push / pskv_pull (ordinary buffers): "
              "push %.1f GB/s, pull %.1f GB/s\n", gib, gib * 1.073741824 / best_push, gib * 1.073741824 / best_pull);
  pskv_table_destroy(t);
}

static void RunFailures(int num_servers) {
  KVWorker<float> kv(0, 1);
  kv.set_slicer(pskv::GpuSlicer<float>(0));
  // the top keys are covered by no server range (src/postoffice.cc:169-180): kv_app.h:542 fails
  std::vector<Key> keys = {5, kMaxKey - 1};
  std::vector<float> vals = {1.0f, 2.0f};
  if ((kMaxKey / num_servers) * num_servers <= kMaxKey - 1) {
    bool thrown = false;
    try {
      kv.Push(keys, vals);
    } catch (const dmlc::Error& e) {
      thrown = true;
      std::printf("expected failure: %s\n", e.what());
    }
    EXPECT(thrown);
  }
  // 3 values for 2 keys: kv_app.h:549
  bool thrown = false;
  try {
    kv.Push({5, 6}, {1.0f, 2.0f, 3.0f});
  } catch (const dmlc::Error&) {
    thrown = true;
  }
  EXPECT(thrown);
}

int main(int argc, char** argv) {
  const int num_servers = argc > 1 ? std::atoi(argv[1]) : 1;
  try {
    Postoffice::Get()->set_num_servers(num_servers);
    auto s0 = StartServers(0, num_servers, PSKV_MODE_SCALAR);
    auto s1 = StartServers(1, num_servers, PSKV_MODE_FIXED);
    auto s2 = StartServers(2, num_servers, PSKV_MODE_FIXED);
    auto s3 = StartServers(3, num_servers, PSKV_MODE_VARLEN);
    auto s4 = StartServers(4, num_servers, PSKV_MODE_SCALAR);
    RunWorker(0, 1000, true);     // 1,000 keys, all 1.0: pull == 50.0f
    RunWorker(4, 10000, false);   // the reference's own sizes and values, on a fresh store
    RunFixed();
    RunVarLen();
    RunFailures(num_servers);
    RunOrderedMatch();
    RunDeviceBufferContract();
    RunRecordedRequests(num_servers);
    auto s6 = StartServers(6, num_servers, PSKV_MODE_SCALAR);
    RunTwoWorkers(6);
    if (argc > 2) {  // floats per key of the dense run from host memory (4194304 is the configuration's)
      auto s5 = StartServers(5, num_servers, PSKV_MODE_FIXED);
      RunDenseFromHost(static_cast<size_t>(std::atoll(argv[2])));
    }
  } catch (const std::exception& e) {
    std::fprintf(stderr, "unexpected exception: %s\n", e.what());
    return 2;
  }
  if (g_failures) {
    std::fprintf(stderr, "%d expectation(s) failed\n", g_failures.load());
    return 1;
  }
  std::printf("test_kv_app_gpu: ok (%d server%s)\n", num_servers, num_servers == 1 ? "" : "s");
  return 0;
}
