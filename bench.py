#!/usr/bin/env python3
"""Benchmark of the pskv hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]

Workloads (BASELINE.json `configs`):
  sparse_lr (default, configs[1]): every step slices 1,000,000 fresh sorted unique uint64
      keys over 4 server key ranges, pushes each slice into the table of its range
      (find-or-insert + float add) and pulls the same keys back. 20 steps grow the
      store to 20M keys. value = (pushed + pulled keys) / s.
  dense (configs[2]): 64 keys x 4,194,304 float32; a step is one push-accumulate of
      1 GiB followed by one full pull. value = algorithmic GB/s.
  varlen (configs[4]): 2,000,000 keys with lens in {8,16,32,64,128} over 16 ranges; a
      step is one push of all keys followed by a pull with lens. value = keys/s.
  zipf (configs[3]): one table; 8 pushes of 4,000,000 distinct Zipf(1.1)-popular keys of a
      100M-key universe, then one pull of 16,000,000 such keys, most of them absent (the pull
      inserts them). value = (pushed + pulled keys) / s.
Further workloads (not BASELINE configurations):
  sparse_repeat: the same 16,000,000 keys pushed and pulled every step (the shape of the
      reference's own test, tests/test_kv_app.cc:27-41, at the size of a model).
  embed: one table of 8M rows of 64 floats; a step pulls the rows of 1,000,000 keys, another
      random subset every step, and pushes a gradient for the same keys.
  match: the ordered match of two sorted key sets (parallel_kv_match.h:29-120), 12M source
      keys merged into 16M destination keys. value = keys of both sides / s.

Prints ONE JSON line. Inputs are resident in HBM before the clock starts. `value` comes
from exactly K timed steps. `roofline` is the dominant kernel of the workload, timed inside
those same steps: launches carry their own start/stop HIP events on the stream they run on
(hipExtLaunchKernelGGL). A pair of events costs about 15 us of host time per launch (and a
few on the GPU), so the steps are sampled: every fourth step times its launches, for the
workloads with several tables those of ONE table, taken in turn. `cpu_baseline` is the CPU oracle on the same inputs, one thread, on a
bounded sample.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

REPO = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, REPO)
import __graft_entry__ as graft  # noqa: E402

KMAX = (1 << 64) - 1
HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
# Launches that carry their own start/stop events cost host time (about 15 us each) and a
# few microseconds on the GPU, so the timed steps are sampled: every SAMPLE_EVERY-th step
# times its launches (for the many-table workloads: those of one table, taken in turn).
SAMPLE_EVERY = 4  # (--sample-every)

# HBM bytes per launch (read + written) of the dominant kernels come from rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE runs of this very script (a counter run cannot be nested in a timing
# run), scaled by what the same counters read for the 1 GiB copy kernel. The summaries of those
# runs under profiles/ carry one line per kernel and launch shape,
#   traffic_per_launch: kind=<kind> units=<keys or floats per launch> read_bytes=<r> written_bytes=<w>
# and this script reports a figure only when it finds the line for the launch shape it ran.
TRAFFIC_FILES = ("sparse_lr.txt", "dense.txt", "varlen.txt", "zipf.txt", "sparse_repeat.txt", "embed.txt",
                 "match.txt")
_traffic_cache = None


def traffic_table():
    """{(kind, units): (bytes, 'profiles/<file>')} from the committed profile summaries."""
    global _traffic_cache
    if _traffic_cache is None:
        _traffic_cache = {}
        for name in TRAFFIC_FILES:
            path = os.path.join(REPO, "profiles", name)
            if not os.path.exists(path):
                continue
            with open(path) as f:
                for line in f:
                    line = line.strip()
                    if not line.startswith("traffic_per_launch: "):
                        continue
                    kv = dict(item.split("=", 1) for item in line[len("traffic_per_launch: "):].split())
                    key = (kv["kind"], int(kv["units"]))
                    _traffic_cache.setdefault(key, (float(kv["read_bytes"]) + float(kv["written_bytes"]),
                                                    "profiles/" + name))
    return _traffic_cache


TRAFFIC_SOURCES = set()


def traffic(kind, units):
    hit = traffic_table().get((kind, int(units)))
    if hit is None:
        return None
    TRAFFIC_SOURCES.add(hit[1])
    return hit[0]


def host_info():
    """The CPU the baseline ran on and how the oracle was compiled."""
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for l in f:
                if l.startswith("model name"):
                    model = l.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"cpu": model, "logical_cpus": os.cpu_count(), "oracle_flags": "g++ -O3 -std=c++11"}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def unique_sorted_keys(rng, n, limit):
    keys = np.unique(rng.integers(0, limit, size=n + n // 64 + 16, dtype=np.uint64))
    while keys.size < n:
        keys = np.unique(np.concatenate([keys, rng.integers(0, limit, size=n, dtype=np.uint64)]))
    if keys.size > n:
        keys = np.sort(rng.choice(keys, size=n, replace=False))
    return keys


def to_dev(a, dev):
    import torch
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint64:
        a = a.view(np.int64)
    return torch.from_numpy(a).to(dev)


def wake_gpu(dev, seconds=2.0):
    """A fresh box hands over a GPU that has been idle: its first second of work runs slower than
    every later one (the first of several identical runs on a box read 10-25 % low, later ones
    agreed to 2 %). Untimed streaming work of a couple of seconds comes before anything is measured."""
    import torch
    x = torch.zeros(1 << 28, device=dev)
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            x.add_(1.0)
        torch.cuda.synchronize()
    del x
    torch.cuda.empty_cache()


def sampled(j, steps):
    """Whether timed step j (0-based) is one whose launches carry events: every SAMPLE_EVERY-th,
    and no more than that share of a short run (but the first step always)."""
    return j >= 0 and j % SAMPLE_EVERY == 0 and j // SAMPLE_EVERY < max(1, steps // SAMPLE_EVERY)


def kernel_stats(tables, kernel):
    """(launches, summed ms, per-launch ms) of one kernel over several tables."""
    n, ms, samples = 0, 0.0, []
    for t in tables:
        a, b = t.prof_read(kernel)
        n += a
        ms += b
        samples.append(t.prof_samples(kernel))
    return n, ms, np.concatenate(samples) if samples else np.zeros(0, np.float32)


def pull_entries(units, pull, same, per_key, traffic_plain, traffic_per_key=None):
    """The `kernels` entries of a SCALAR pull. Once a table has seen pulls come right behind pushes
    of the same keys, the pushes leave their keys and values behind in request order and such a
    pull compares and answers in one pass over them (24 B/key, all of it streamed). A pull that
    repeats a key set whose values have run ahead of the slots is decided as a whole first: the
    keys are compared by k_same_keys (16 B/key) and the pull kernel streams the values (8 B/key).
    Any other pull goes through the slots (24 B/key algorithmic, a 128-byte line per key)."""
    out = {}
    cached = same[0] > 0
    if per_key[0]:
        out["pull_scalar"] = dict(roofline(24.0 * units, per_key[0], per_key[1], traffic_per_key, per_key[2]),
                                  bytes_per_key=24,
                                  path="compared with the keys the push left behind and answered from its "
                                       "values, one pass")
        if pull[0]:
            out["pull_scalar_other"] = dict(roofline(24.0 * units, pull[0], pull[1], None, pull[2]),
                                            bytes_per_key=24,
                                            path="the other pulls of the run: through the slots" +
                                                 (", or streamed from the key cache behind k_same_keys" if cached
                                                  else ""))
    else:
        out["pull_scalar"] = dict(roofline((8.0 if cached else 24.0) * units, pull[0], pull[1],
                                           None if cached else traffic_plain, pull[2]),
                                  bytes_per_key=8 if cached else 24,
                                  path="served from the key cache (k_same_keys in front)" if cached
                                       else "through the slots")
    if cached:
        out["same_keys"] = dict(roofline(16.0 * units, same[0], same[1], None, same[2]), bytes_per_key=16,
                                kernel="k_same_keys (request keys against cached keys)")
    return out


def roofline(alg_bytes_per_launch, launches, total_ms, traffic=None, samples=None):
    """`achieved` is algorithmic bytes over the AVERAGE launch duration; the median and the
    minimum over the launches are given beside it."""
    if not launches:
        raise RuntimeError("no timed launch of the kernel: its events were switched off")
    avg_s = total_ms / launches * 1e-3
    achieved = alg_bytes_per_launch / avg_s / 1e9
    r = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
         "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
         "launches": launches, "avg_us": round(avg_s * 1e6, 2),
         "alg_bytes_per_launch": int(alg_bytes_per_launch)}
    if samples is not None and len(samples):
        r["median_us"] = round(float(np.median(samples)) * 1e3, 2)
        r["min_us"] = round(float(np.min(samples)) * 1e3, 2)
    return r


# ------------------------------------------------------------------------------------
# sparse_lr: configs[1]
# ------------------------------------------------------------------------------------
def gen_sparse_lr(steps, n, S):
    limit = (KMAX // S) * S  # keys the stock ranges cover (postoffice.cc:169-180)
    batches = []
    for p in range(steps):
        rng = np.random.default_rng(0xC0FFEE + p)
        keys = unique_sorted_keys(rng, n, limit)
        vals = rng.normal(0.0, 0.01, size=n).astype(np.float32)
        batches.append((keys, vals))
    return batches


def run_sparse_lr(args, capi, dev):
    import torch
    n, S = args.keys or 1000000, 4
    total_steps = args.warmup + args.steps
    log("generating %d batches of %d keys" % (total_steps, n))
    batches = gen_sparse_lr(total_steps, n, S)
    rb, re = capi.server_ranges(S)
    d_batches = [(to_dev(k, dev), to_dev(v, dev)) for k, v in batches]
    out = torch.empty(n, dtype=torch.float32, device=dev)
    # One table per server key range. The tables share one stream: their kernels run back to
    # back, each with the whole GPU, so a kernel's duration is its own and not that of four
    # overlapping launches.
    stream = torch.cuda.Stream()
    last = total_steps - 1
    want = batches[last][1] + np.float32(0.0)  # each key was pushed once: 0.0f + v

    def measure(cap, per_table, sample, own_streams=False):
        """The warm-up and the timed steps on fresh tables of `cap` keys each (0: the library's
        default, tables that grow while the clock runs). Returns seconds and kernel statistics."""
        if own_streams:
            tables = [capi.Table(capi.MODE_SCALAR, initial_capacity=cap) for _ in range(S)]
            group = None
        else:
            group = capi.Group(S, capi.MODE_SCALAR, initial_capacity=cap, stream=stream.cuda_stream)
            tables = group.tables
        prof_on = [-1]  # the table whose launches carry events at the moment (-1: none)

        def step(i):
            # Kernel durations are sampled INSIDE the timed steps: in every SAMPLE_EVERY-th step the
            # launches carry their own start/stop events (booked to the first table of the group; with
            # one call per table those of one of the S tables, taken in turn). Events on every launch
            # would cost more host time per step than the GPU needs for it.
            if sample:
                j = i - args.warmup
                on = sampled(j, args.steps)
                which = ((j // SAMPLE_EVERY) % S if per_table else 0) if on else -1
                if which != prof_on[0]:
                    for s_ in range(S):
                        tables[s_].prof_enable(s_ == which)
                    prof_on[0] = which
            dk, dv = d_batches[i]
            # Every step slices its keys, pushes and pulls, in line. (Slicing the keys of coming steps
            # ahead of time, on this thread or on a second one, was measured and gains nothing: the
            # slicer's short kernel shares the GPU with the store's long ones either way.)
            pos, _, used = capi.slice_keys(dk, rb, re, nvals=n)
            kp, vp, op = dk.data_ptr(), dv.data_ptr(), out.data_ptr()
            if not per_table:
                # one launch per step of the pipeline over all S key ranges
                group.push_raw(kp, pos, vp, pos)
                group.pull_raw(kp, pos, op)
                return
            pos = [int(x) for x in pos]
            for s_ in range(S):
                if used[s_]:
                    c = pos[s_ + 1] - pos[s_]
                    tables[s_].push_raw(kp + 8 * pos[s_], c, vp + 4 * pos[s_], c)
            for s_ in range(S):
                if used[s_]:
                    c = pos[s_ + 1] - pos[s_]
                    tables[s_].pull_raw(kp + 8 * pos[s_], c, op + 4 * pos[s_], c)

        def drain():
            if per_table:
                for t in tables:
                    t.sync()
            else:
                group.sync()
            torch.cuda.synchronize()

        for i in range(args.warmup):
            step(i)
        drain()
        for t in tables:
            t.prof_reset()
        t0 = time.perf_counter()
        for i in range(args.warmup, total_steps):
            step(i)
        drain()
        dt = time.perf_counter() - t0
        st = {"push": kernel_stats(tables, capi.KERNEL_PUSH_SCALAR),
              "pull": kernel_stats(tables, capi.KERNEL_PULL_SCALAR),
              "same": kernel_stats(tables, capi.KERNEL_SAME_KEYS),
              "per_key": kernel_stats(tables, capi.KERNEL_PULL_PER_KEY),
              "growth": kernel_stats(tables, capi.KERNEL_REHASH)}
        for t in tables:
            t.prof_enable(False)
        # the last pull must hold exactly the pushed values, the tables every key of the run
        got = out.cpu().numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), "pulled values differ"
        held = sum(t.size()[0] for t in tables)
        assert held == n * total_steps, (held, n * total_steps)
        if group is not None:
            group.close()
        else:
            for t in tables:
                t.close()
        return dt, st, held

    per_table = args.per_table
    cap_presized = int(n * (args.warmup + 2 * args.steps) / S * 1.1)
    # An untimed rehearsal of the whole run on tables of its own, closed before the measured ones are
    # created. It changes nothing in the library (fresh tables start from the same state) but the state
    # of the GPU's memory: the first time a process grows its tables it is handed memory that the
    # previous process on the box may have left unwiped, and right after a process that churned tens of
    # GB the growths then cost 10-25 % of the run (0.128-0.145 ms/step against 0.118; the second run
    # of a process takes 0.114-0.119 wherever it starts). A figure that depends on the previous tenant
    # of the box measures the box.
    if not args.no_rehearsal:
        measure(0, per_table, False)
    # THE measured run: tables created with the library's defaults (room for 1M keys each), which
    # grow while the clock runs, as the std::unordered_map of the reference's handle does (kv_app.h:462)
    dt, st, held = measure(0, per_table, True)
    keys_per_launch = n / S if per_table else n
    res = {
        "value": 2.0 * n * args.steps / dt, "unit": "keys/s", "ms_per_step": dt / args.steps * 1e3,
        "dtype": "f32",
        "config": {"workload": "sparse_lr: 1M sorted unique uint64 keys/step over 4 key ranges, "
                               "push then pull, store grows by 1M keys/step; tables created with the "
                               "default capacity, their growths inside the timed steps", "keys_per_step": n,
                   "rehearsal": "none" if args.no_rehearsal else
                                "one untimed run of the same steps on tables of its own, closed before the measured "
                                "tables are created",
                   "ranges": S, "value_len": 1, "key_dtype": "u64",
                   "store_keys_after_timed_steps": held,
                   "launches": "one launch per table" if per_table else
                               "one launch over all %d key ranges (pskv_push_multi / pskv_pull_multi)" % S},
        # every pushed key is new: 8 key + 4 val in, 8 slot read, 8 key + 4 val written
        "roofline": dict(roofline(32.0 * keys_per_launch, st["push"][0], st["push"][1],
                                  traffic("push_scalar", keys_per_launch), st["push"][2]),
                         kernel="k_scalar<push> (find-or-insert + add)", bytes_per_key=32),
        "kernels": dict(pull_entries(keys_per_launch, st["pull"], st["same"], st["per_key"],
                                     traffic("pull_scalar", keys_per_launch),
                                     traffic("pull_per_key", keys_per_launch)),
                        growth={"launches": st["growth"][0], "total_us": round(st["growth"][1] * 1e3, 1),
                                "note": "k_regrow + k_regrow_rest of the sampled steps only"}),
    }
    if not args.no_extra:
        # the same steps on tables sized up front for every key of the run (no growth, lower fill)
        dt_p, st_p, _ = measure(cap_presized, per_table, True)
        res["presized"] = {"value": 2.0 * n * args.steps / dt_p, "unit": "keys/s",
                           "ms_per_step": dt_p / args.steps * 1e3,
                           "push_kernel": roofline(32.0 * keys_per_launch, st_p["push"][0], st_p["push"][1],
                                                   traffic("push_scalar", keys_per_launch), st_p["push"][2]),
                           "note": "same steps on tables created with room for %d keys each: no growth "
                                   "inside the timed steps, fill below 0.2" % cap_presized}
        # ... and with one call per table, which is what S separate KVServers on one GPU would issue
        dt_t, _, _ = measure(0, not per_table, False)
        res["per_table" if not per_table else "multi"] = {
            "value": 2.0 * n * args.steps / dt_t, "unit": "keys/s", "ms_per_step": dt_t / args.steps * 1e3,
            "note": "same steps, default-capacity tables, " +
                    ("one pskv_push / pskv_pull per table" if not per_table else
                     "one pskv_push_multi / pskv_pull_multi over all ranges")}
    # On request, the same timed steps once more on fresh tables that keep the library's default
    # of one stream per table: kernels of different key ranges then overlap, so whole-job
    # throughput is higher, but a kernel's duration is no longer its own, which is why the
    # headline figures come from the shared-stream run.
    if args.own_streams:
        dt_own, _, _ = measure(0, True, False, own_streams=True)
        res["own_streams"] = {"value": 2.0 * n * args.steps / dt_own, "unit": "keys/s",
                              "ms_per_step": dt_own / args.steps * 1e3,
                              "note": "same steps, one stream per table (kernels of different ranges overlap)"}
    # the slicer alone on an idle GPU: one launch and one read-back of S+1 positions
    t_s = time.perf_counter()
    for _ in range(50):
        capi.slice_keys(d_batches[0][0], rb, re, nvals=n)
    slice_us = (time.perf_counter() - t_s) / 50 * 1e6
    res["kernels"]["slicer"] = {"wall_us_per_call": round(slice_us, 1), "keys": n, "ranges": S}
    return res, batches[args.warmup:args.warmup + args.steps], (n, S)


def cpu_sparse_lr(orc, batches, n, S, budget_s=25.0):
    rb, re = orc.server_ranges(S)
    stores = [orc.Store(orc.MODE_SCALAR) for _ in range(S)]
    done = 0
    t0 = time.perf_counter()
    for keys, vals in batches:
        pos, _, used = orc.slice_keys(keys, rb, re, nvals=n)
        pos = pos.astype(np.int64)
        for s in range(S):
            if used[s]:
                stores[s].push(keys[pos[s]:pos[s + 1]], vals[pos[s]:pos[s + 1]])
        for s in range(S):
            if used[s]:
                stores[s].handle(False, True, keys[pos[s]:pos[s + 1]], out_cap=int(pos[s + 1] - pos[s]))
        done += 1
        if time.perf_counter() - t0 > budget_s:
            break
    dt = time.perf_counter() - t0
    return {"value": 2.0 * n * done / dt, "unit": "keys/s", "cores": 1, "kind": "port",
            "sample": "first %d of the timed steps (slice + push + pull of %d keys each), "
                      "std::unordered_map store per range, one thread; the maps start empty and rehash as "
                      "they grow inside this timing, as the GPU tables of `value` do" % (done, n)}


# ------------------------------------------------------------------------------------
# dense: configs[2]
# ------------------------------------------------------------------------------------
def measure_dense(capi, dev, steps, warmup, nk=64, k=4194304, every_step=False):
    """Returns (seconds for `steps` push+pull steps, accumulate stats, gather stats)."""
    import torch
    keys = to_dev(np.uint64(KMAX // nk) * np.arange(nk, dtype=np.uint64), dev)
    g = torch.Generator(device=dev)
    g.manual_seed(0xD15E)
    vals = torch.rand(nk * k, device=dev, generator=g) * 2 - 1
    out = torch.empty(nk * k, dtype=torch.float32, device=dev)
    t = capi.Table(capi.MODE_FIXED, initial_capacity=1024, row_len=k, arena_floats=nk * k)
    t.push(keys, vals)  # first touch creates the rows
    for _ in range(warmup):
        t.push(keys, vals)
        t.pull(keys, out)
    t.sync()
    torch.cuda.synchronize()
    # the launches of every SAMPLE_EVERY-th timed step carry their own HIP events
    t.prof_enable(True)
    t.prof_reset()
    t0 = time.perf_counter()
    for i in range(steps):
        t.prof_enable(every_step or sampled(i, steps))  # (15 us of events next to 500 us kernels)
        t.push(keys, vals)
        t.pull(keys, out)
    t.sync()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    acc = kernel_stats([t], capi.KERNEL_ROWS_ACC)
    gat = kernel_stats([t], capi.KERNEL_ROWS_GATHER)
    # closed form: every float holds (1 + warmup + steps) * v, accumulated one add at a time
    idx = torch.randint(0, nk * k, (4096,), device=dev)
    ref = torch.zeros(4096, device=dev)
    for _ in range(1 + warmup + steps):
        ref = ref + vals[idx]
    assert torch.equal(out[idx], ref), "dense sums differ from sequential float adds"
    # plain copies of the same 1 GiB: the known-size launch that memory-traffic counters are
    # scaled by, and the copy ceiling of this GPU next to the accumulate kernel
    t.prof_enable(True)  # the last timed step may have left the events off
    for _ in range(3):
        t.copy_probe(out, vals)
    t.sync()
    cp = kernel_stats([t], capi.KERNEL_COPY)
    t.prof_enable(False)
    t.close()
    return dt, acc, gat, cp, nk, k


def run_dense(args, capi, dev):
    dt, acc, gat, cp, nk, k = measure_dense(capi, dev, args.steps, args.warmup)
    floats = nk * k
    res = {
        "value": 20.0 * floats * args.steps / dt / 1e9, "unit": "GB/s",
        "ms_per_step": dt / args.steps * 1e3, "dtype": "f32",
        "config": {"workload": "dense: 64 keys x 4,194,304 f32 (1 GiB), push-accumulate then full pull",
                   "keys_per_step": nk, "value_len": k},
        # 4 B in + 4 B row read + 4 B row write per float
        "roofline": dict(roofline(12.0 * floats, acc[0], acc[1], traffic("rows_acc_fixed", floats), acc[2]),
                         kernel="k_rows<acc,fixed> (row += in)", bytes_per_float=12),
        "kernels": {"rows_gather": dict(roofline(8.0 * floats, gat[0], gat[1],
                                                 traffic("rows_gather_fixed", floats), gat[2]),
                                        bytes_per_float=8),
                    "copy_ceiling": dict(roofline(8.0 * floats, cp[0], cp[1], 8.0 * floats, cp[2]),
                                         kernel="k_copy (plain copy of the same 1 GiB)")},
    }
    return res


def cpu_dense(orc, nk=64, k=4194304, sample_keys=16, budget_s=10.0):
    rng = np.random.default_rng(0xD15E)
    keys = (np.uint64(KMAX // nk) * np.arange(sample_keys, dtype=np.uint64))
    vals = rng.uniform(-1, 1, size=sample_keys * k).astype(np.float32)
    st = orc.Store(orc.MODE_FIXED, k)
    st.push(keys, vals)
    t0 = time.perf_counter()
    reps = 0
    while reps < 3 or time.perf_counter() - t0 < budget_s:
        st.push(keys, vals)
        st.handle(False, True, keys, out_cap=vals.size)
        reps += 1
    dt = time.perf_counter() - t0
    return {"value": 20.0 * vals.size * reps / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "%d of the 64 rows (%d MiB), %d push+pull steps, one thread" % (
                sample_keys, vals.size * 4 >> 20, reps)}


# ------------------------------------------------------------------------------------
# varlen: configs[4]
# ------------------------------------------------------------------------------------
def timed_replays(rec, group, steps, ref, add):
    """Times `steps` runs of a recorded push + pull step (after two untimed ones). `ref` holds the sums a
    sample of the values has reached; every application of the step adds `add` to it. Returns the entry
    for the result line and the sums the sample must have reached."""
    ref = ref + add  # recording a request serves it once
    for _ in range(2):
        rec.run()
        ref = ref + add
    group.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        rec.run()
    t_host = time.perf_counter() - t0
    group.sync()
    dt = time.perf_counter() - t0
    for _ in range(steps):
        ref = ref + add
    return {"ms_per_step": dt / steps * 1e3, "host_us_per_step": t_host / steps * 1e6,
            "note": "the same step kept as a HIP graph by pskv_replay_record and applied by pskv_replay_run: "
                    "one call, one launch, nothing sliced, allocated or waited for per step"}, ref


def with_rates(replayed, n):
    """Adds keys/s (pushed + pulled keys per step) to a `replayed` entry and to its `as_launches` part."""
    out = dict(replayed, value=2.0 * n / (replayed["ms_per_step"] * 1e-3), unit="keys/s")
    out["as_launches"] = dict(replayed["as_launches"], value=2.0 * n / (replayed["as_launches"]["ms_per_step"] * 1e-3),
                              unit="keys/s")
    return out


def replay_both(capi, group, steps, ref, add, *record_args):
    """Records the push + pull step with `record_args` (after the flags) as a HIP graph and as its launches,
    times `steps` runs of each; returns the `replayed` entry and the sums the sample must have reached."""
    rec = group.record(capi.REPLAY_PUSH | capi.REPLAY_PULL, *record_args)
    replayed, ref = timed_replays(rec, group, steps, ref, add)
    rec.close()
    rec = group.record(capi.REPLAY_PUSH | capi.REPLAY_PULL | capi.REPLAY_LAUNCHES, *record_args)
    relaunched, ref = timed_replays(rec, group, steps, ref, add)
    rec.close()
    relaunched["note"] = ("the same recording kept as its launches (PSKV_REPLAY_LAUNCHES), made again one by one by "
                          "pskv_replay_run")
    replayed["as_launches"] = relaunched
    return replayed, ref


def gen_varlen(n, S):
    limit = (KMAX // S) * S
    keys = unique_sorted_keys(np.random.default_rng(0xE3B), n, limit)
    lens = np.random.default_rng(0xE3C).choice(np.array([8, 16, 32, 64, 128], np.int32), size=n)
    return keys, lens.astype(np.int32)


def run_varlen(args, capi, dev):
    import torch
    n, S = args.keys or 2000000, 16
    keys, lens = gen_varlen(n, S)
    nvals = int(lens.sum())
    rb, re = capi.server_ranges(S)
    dk, dl = to_dev(keys, dev), to_dev(lens, dev)
    g = torch.Generator(device=dev)
    g.manual_seed(0xE3D)
    dv = torch.randn(nvals, device=dev, generator=g) * 0.1
    out = torch.empty(nvals, dtype=torch.float32, device=dev)
    out_lens = torch.empty(n, dtype=torch.int32, device=dev)
    torch.cuda.synchronize()  # the raw-pointer calls below do not wait for torch's stream
    stream = torch.cuda.Stream()  # one stream for all ranges: kernels run one at a time
    group = capi.Group(S, capi.MODE_VARLEN, initial_capacity=int(n / S * 1.2) * 4,
                       arena_floats=int(nvals / S * 1.5) + 8 * n // S, stream=stream.cuda_stream)
    tables = group.tables
    per_table = args.per_table
    kp, vp, lp, op, olp = dk.data_ptr(), dv.data_ptr(), dl.data_ptr(), out.data_ptr(), out_lens.data_ptr()

    def step():
        pos, vpos, used = capi.slice_keys(dk, rb, re, lens=dl, nvals=nvals)
        if not per_table:
            # one launch per step of the pipeline over all S key ranges
            group.push_raw(kp, pos, vp, vpos, lp)
            group.pull_raw(kp, pos, op, vpos, olp)
            return
        pos, vpos = [int(x) for x in pos], [int(x) for x in vpos]
        for s in range(S):
            if used[s]:
                c, f = pos[s + 1] - pos[s], vpos[s + 1] - vpos[s]
                tables[s].push_raw(kp + 8 * pos[s], c, vp + 4 * vpos[s], f, lp + 4 * pos[s], c)
        for s in range(S):
            if used[s]:
                c, f = pos[s + 1] - pos[s], vpos[s + 1] - vpos[s]
                tables[s].pull_raw(kp + 8 * pos[s], c, op + 4 * vpos[s], f, olp + 4 * pos[s])

    def drain():
        if per_table:
            for t in tables:
                t.sync()
        else:
            group.sync()
        torch.cuda.synchronize()

    step()  # creates the rows
    for _ in range(args.warmup):
        step()
    drain()
    for t in tables:
        t.prof_reset()
    t0 = time.perf_counter()
    for i in range(args.steps):
        # kernel durations are sampled inside the timed steps: in every SAMPLE_EVERY-th step the
        # launches carry their own events (with --per-table those of one table, taken in turn)
        for s in range(S):
            tables[s].prof_enable(sampled(i, args.steps) and
                                  s == ((i // SAMPLE_EVERY) % S if per_table else 0))
        step()
    drain()
    dt = time.perf_counter() - t0
    acc = kernel_stats(tables, capi.KERNEL_ROWS_ACC)
    gat = kernel_stats(tables, capi.KERNEL_ROWS_GATHER)
    for t in tables:
        t.prof_enable(False)
    assert torch.equal(out_lens, dl), "pulled lens differ"
    idx = torch.randint(0, nvals, (4096,), device=dev)
    ref = torch.zeros(4096, device=dev)
    for _ in range(1 + args.warmup + args.steps):
        ref = ref + dv[idx]
    assert torch.equal(out[idx], ref), "var-len sums differ from sequential float adds"
    replayed = None
    if not per_table:
        # the same step recorded once (pskv_replay_record) and replayed: no slicing, one call and one launch
        pos, vpos, _ = capi.slice_keys(dk, rb, re, lens=dl, nvals=nvals)
        replayed, ref = replay_both(capi, group, args.steps, ref, dv[idx], dk, pos, dv, vpos, dl, out, vpos, out_lens)
        assert torch.equal(out_lens, dl), "pulled lens differ"
        assert torch.equal(out[idx], ref), "replayed var-len sums differ from sequential float adds"
    # on request, once more with the library's default of one stream per table (launches of
    # different ranges overlap; durations are then no longer a kernel's own, hence not the headline)
    dt_own = None
    if args.own_streams:
        group.close()
        tables = [capi.Table(capi.MODE_VARLEN, initial_capacity=int(n / S * 1.2) * 4,
                             arena_floats=int(nvals / S * 1.5) + 8 * n // S) for _ in range(S)]
        per_table = True  # tables with streams of their own go one by one
        step()
        for _ in range(args.warmup):
            step()
        drain()
        t1 = time.perf_counter()
        for _ in range(args.steps):
            step()
        drain()
        dt_own = time.perf_counter() - t1
        assert torch.equal(out_lens, dl), "pulled lens differ"
    floats_per_launch = nvals / S if args.per_table else nvals
    res = {
        "value": 2.0 * n * args.steps / dt, "unit": "keys/s", "ms_per_step": dt / args.steps * 1e3,
        "dtype": "f32",
        "config": {"workload": "varlen: 2M keys, lens in {8,16,32,64,128}, 16 key ranges, push then "
                               "pull with lens", "keys_per_step": n, "floats_per_step": nvals, "ranges": S,
                   "launches": "one launch per table" if args.per_table else
                               "one launch over all %d key ranges (pskv_push_multi / pskv_pull_multi)" % S},
        "gbps": (20.0 * nvals + 56.0 * n) * args.steps / dt / 1e9,
        "roofline": dict(roofline(12.0 * floats_per_launch, acc[0], acc[1],
                                  traffic("rows_acc_varlen", floats_per_launch), acc[2]),
                         kernel="k_rows<acc,varlen> (row += in)", bytes_per_float=12),
        "kernels": {"rows_gather": dict(roofline(8.0 * floats_per_launch, gat[0], gat[1],
                                                 traffic("rows_gather_varlen", floats_per_launch), gat[2]),
                                        bytes_per_float=8)},
    }
    if replayed is not None:
        res["replayed"] = with_rates(replayed, n)
    if dt_own is not None:
        res["own_streams"] = {"value": 2.0 * n * args.steps / dt_own, "unit": "keys/s",
                              "ms_per_step": dt_own / args.steps * 1e3,
                              "gbps": (20.0 * nvals + 56.0 * n) * args.steps / dt_own / 1e9,
                              "note": "same steps, one stream per table (kernels of different ranges overlap)"}
    return res, (keys, lens, nvals, n, S)


def cpu_dense_all_cores(orc, threads=16, nk=64, k=4194304, budget_s=8.0):
    """The same row loop sharded by key over `threads` host threads, each with a store of its
    own (keys are independent, so this is how a multi-threaded CPU server would split the
    work). Labelled as such: the reference runs its handle on one thread."""
    import threading
    per = nk // threads
    rng = np.random.default_rng(0xD15E)
    vals = rng.uniform(-1, 1, size=per * k).astype(np.float32)  # every thread pushes the same floats
    stores, keysets = [], []
    for t in range(threads):
        keys = np.uint64(KMAX // nk) * np.arange(t * per, (t + 1) * per, dtype=np.uint64)
        st = orc.Store(orc.MODE_FIXED, k)
        st.push(keys, vals)
        stores.append(st)
        keysets.append(keys)
    counts = [0] * threads
    stop = time.perf_counter() + budget_s

    def work(t):
        while time.perf_counter() < stop:
            stores[t].push(keysets[t], vals)
            stores[t].handle(False, True, keysets[t], out_cap=vals.size)
            counts[t] += 1

    ths = [threading.Thread(target=work, args=(t,)) for t in range(threads)]
    t0 = time.perf_counter()
    for th in ths:
        th.start()
    for th in ths:
        th.join()
    dt = time.perf_counter() - t0
    return {"value": 20.0 * vals.size * sum(counts) / dt / 1e9, "unit": "GB/s", "cores": threads,
            "kind": "port", "sample": "all-core variant: %d threads, each push + pull of %d rows of %d "
                                      "floats into its own store, %d steps in total" % (threads, per, k, sum(counts))}


def cpu_varlen(orc, keys, lens, nvals, n, S, budget_s=15.0):
    rng = np.random.default_rng(0xE3D)
    vals = rng.normal(0, 0.1, size=nvals).astype(np.float32)
    rb, re = orc.server_ranges(S)
    st = orc.Store(orc.MODE_VARLEN)  # the ranges are disjoint: one store serves all of them
    pos, vpos, used = orc.slice_keys(keys, rb, re, lens, nvals)
    st.push(keys, vals, lens)
    done = 0
    t0 = time.perf_counter()
    while done < 2 or time.perf_counter() - t0 < budget_s:
        orc.slice_keys(keys, rb, re, lens, nvals)
        st.push(keys, vals, lens)
        st.handle(False, True, keys, out_cap=nvals)
        done += 1
    dt = time.perf_counter() - t0
    return {"value": 2.0 * n * done / dt, "unit": "keys/s", "cores": 1, "kind": "port",
            "sample": "%d full steps (slice + push + pull of %d keys, %d floats), one thread" % (done, n, nvals)}


# ------------------------------------------------------------------------------------
# zipf: configs[3]
# ------------------------------------------------------------------------------------
_zipf_weights = {}


def zipf_distinct_ranks(rng, n, universe, s=1.1):
    """The n distinct ranks of [0, universe) that a long run of Zipf(s) draws over the universe
    names, sorted. Drawing rank after rank until n distinct ones have come up takes about 45
    draws per key at these sizes (minutes of host time for the 16M-key pull); the shortcut: D
    draws name rank k at least once with probability 1 - exp(-D p_k), independently for every k
    when the number of draws is Poisson, so one exponential variate per rank, compared with
    D p_k, gives the set of named ranks directly. D is aimed so that about n ranks come up; the
    set is then thinned at random, or topped up with further draws by popularity, to exactly n."""
    key = (universe, s)
    if key not in _zipf_weights:
        w = np.power(np.arange(1, universe + 1, dtype=np.float32), np.float32(-s))
        _zipf_weights.clear()
        _zipf_weights[key] = (w / np.float32(w.sum(dtype=np.float64)), np.cumsum(w[::1024], dtype=np.float64))
    p, _ = _zipf_weights[key]
    sub = p[::97].astype(np.float64)  # the expected count on a thinned copy is close enough to aim with
    lo, hi = 1.0, 1e13
    for _ in range(60):
        d = (lo * hi) ** 0.5
        if (1.0 - np.exp(-d * sub)).sum() * 97 < n * 1.002:
            lo = d
        else:
            hi = d
    e = rng.standard_exponential(universe, dtype=np.float32)
    ranks = np.flatnonzero(e < np.float32(hi) * p)
    del e
    while ranks.size < n:
        more = (rng.zipf(s, size=4 * (n - ranks.size) + 1024) - 1)
        ranks = np.unique(np.concatenate([ranks, more[(more >= 0) & (more < universe)]]))
    if ranks.size > n:
        ranks = np.sort(rng.choice(ranks, size=n, replace=False))
    return ranks


def rank_to_key(ranks):
    """An injective scatter of ranks over the covered key space (odd multiplier mod 2^64, then >> 1)."""
    return (ranks.astype(np.uint64) * np.uint64(0x9E3779B97F4A7C15)) >> np.uint64(1)


def gen_zipf(pushes, n_push, n_pull, universe):
    """The inputs of configs[3]: `pushes` worker requests of n_push distinct Zipf(1.1)-popular keys
    with N(0,1) values, and the n_pull distinct Zipf-popular keys of the pull."""
    batches = []
    for w in range(pushes):
        rng = np.random.default_rng(0x21F + w)
        keys = np.sort(rank_to_key(zipf_distinct_ranks(rng, n_push, universe)))
        batches.append((keys, rng.standard_normal(n_push).astype(np.float32)))
    rng = np.random.default_rng(0x9011)
    probe = np.sort(rank_to_key(zipf_distinct_ranks(rng, n_pull, universe)))
    _zipf_weights.clear()  # (400 MB)
    return batches, probe


def run_zipf(args, capi, dev, pushes=8):
    """configs[3] as it stands: 8 worker pushes of 4M distinct Zipf-popular keys each into one table
    (a growing share of every push is already stored), applied in order, then ONE pull of 16M
    distinct Zipf-popular keys, most of which the store has never seen and which the pull inserts
    with value 0 (kv_app.h:456-458). The table starts at the default capacity and grows inside the
    timed region as it would in service. The clock covers the 8 pushes and the pull."""
    import torch
    n, universe = args.keys or 4000000, 100000000
    n_pull = 4 * n
    log("generating %d Zipf batches of %d keys and a pull of %d" % (pushes, n, n_pull))
    batches, probe = gen_zipf(pushes, n, n_pull, universe)
    d_batches = [(to_dev(k, dev), to_dev(v, dev)) for k, v in batches]
    d_probe = to_dev(probe, dev)
    out = torch.empty(n_pull, dtype=torch.float32, device=dev)
    torch.cuda.synchronize()

    def once(prof):
        t = capi.Table(capi.MODE_SCALAR)
        t.prof_enable(prof)  # one launch per request: per-launch events cost nothing that matters here
        t.sync()
        t0 = time.perf_counter()
        for dk, dv in d_batches:
            t.push(dk, dv)
        t.sync()
        t1 = time.perf_counter()
        t.pull(d_probe, out)
        t.sync()
        t2 = time.perf_counter()
        return t, t1 - t0, t2 - t1

    for _ in range(max(1, min(args.warmup, 2))):  # whole runs on tables of their own: the first one loads the code
        t, _, _ = once(False)
        t.close()
    t, dt_push, dt_pull = once(True)
    push = kernel_stats([t], capi.KERNEL_PUSH_SCALAR)
    pull = kernel_stats([t], capi.KERNEL_PULL_SCALAR)
    rehash = kernel_stats([t], capi.KERNEL_REHASH)
    held = t.size()[0]
    everything = np.unique(np.concatenate([k for k, _ in batches] + [probe]))
    assert held == everything.size, (held, everything.size)
    # spot check against sequential float adds in push order: 4096 pulled keys
    pick = np.random.default_rng(5).choice(n_pull, size=4096, replace=False)
    want = np.zeros(4096, np.float32)
    for keys, vals in batches:
        at = np.minimum(np.searchsorted(keys, probe[pick]), keys.size - 1)
        hit = keys[at] == probe[pick]
        want[hit] = want[hit] + vals[at[hit]]
    got = out.cpu().numpy()[pick]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), "pulled values differ"
    stored_before = np.unique(np.concatenate([k for k, _ in batches]))
    missing = n_pull - int(np.isin(probe, stored_before, assume_unique=True).sum())
    t.close()
    dt = dt_push + dt_pull
    total_keys = pushes * n + n_pull
    res = {
        "value": total_keys / dt, "unit": "keys/s", "ms_per_step": dt / pushes * 1e3,
        "dtype": "f32",
        "config": {"workload": "zipf: %d pushes of 4M distinct Zipf(1.1)-popular keys from a 100M-key universe "
                               "into one table that starts at the default capacity, then one pull of 16M "
                               "distinct Zipf-popular keys (%d of them absent: inserted with value 0); a step "
                               "is one push, the pull's time is spread over the steps" % (pushes, missing),
                   "keys_per_step": n, "pull_keys": n_pull, "pull_keys_absent": missing, "ranges": 1,
                   "value_len": 1, "key_dtype": "u64", "store_keys_at_the_end": held},
        "phases": {"pushes_ms": dt_push * 1e3, "pull_ms": dt_pull * 1e3,
                   "push_keys_per_s": pushes * n / dt_push, "pull_keys_per_s": n_pull / dt_pull},
        # a pulled key that is absent: 8 key in, 8 slot read, 8 key written, 4 out = 28 B/key; the present
        # ones read the value instead of writing the key: 24 B/key; priced as misses
        "roofline": dict(roofline(28.0 * n_pull, pull[0], pull[1], traffic("pull_miss_insert", n_pull), pull[2]),
                         kernel="k_scalar<pull> (find, or insert 0, then answer), %d of %d keys absent" % (missing, n_pull),
                         bytes_per_key=28),
        # between a hit (28 B/key) and an insert (32 B/key); priced as inserts
        "kernels": {"push_scalar": dict(roofline(32.0 * n, push[0], push[1], traffic("push_scalar_zipf", n), push[2]),
                                        kernel="k_scalar<push> (find-or-insert + add), 4M keys", bytes_per_key=32),
                    "growth": {"launches": rehash[0], "total_us": round(rehash[1] * 1e3, 1),
                               "kernels": "k_regrow + k_regrow_rest per growth"}},
    }
    return res, (batches, probe)


def cpu_zipf(orc, batches, probe, budget_s=25.0):
    store = orc.Store(orc.MODE_SCALAR)
    done = 0
    t0 = time.perf_counter()
    for keys, vals in batches:
        store.push(keys, vals)
        done += keys.size
        if time.perf_counter() - t0 > budget_s:
            break
    pulled = False
    if done == sum(k.size for k, _ in batches):
        store.handle(False, True, probe, out_cap=probe.size)
        done += probe.size
        pulled = True
    dt = time.perf_counter() - t0
    return {"value": done / dt, "unit": "keys/s", "cores": 1, "kind": "port",
            "sample": "%s on one std::unordered_map store, one thread" % (
                "the same %d pushes and the pull of %d keys" % (len(batches), probe.size) if pulled else
                "the pushes that fit %d s (%d keys), without the pull" % (budget_s, done))}


# ------------------------------------------------------------------------------------
# sparse_repeat: the same key set pushed again and again (the shape of the reference's own
# test, tests/test_kv_app.cc:27-41, at the size of a sparse model)
# ------------------------------------------------------------------------------------
def run_sparse_repeat(args, capi, dev):
    """One SCALAR table; every step pushes the SAME 16M sorted unique keys with fresh values and
    pulls them back. From the third request on the table serves the key set from its
    request-ordered value array: a streamed comparison of the keys, then `cached[i] += v[i]`."""
    import torch
    n = args.keys or 16000000
    rng = np.random.default_rng(0x5EED)
    keys = unique_sorted_keys(rng, n, KMAX)
    vals = rng.normal(0.0, 0.01, size=n).astype(np.float32)
    dk, dv = to_dev(keys, dev), to_dev(vals, dev)
    out = torch.empty(n, dtype=torch.float32, device=dev)
    # Room for the requests in flight: until the device's first records have arrived, the host must
    # assume that a request creates all its keys. (A table created with the default capacity grows to
    # that room by itself during the first requests and then runs the same steps at the same speed.)
    group = capi.Group(1, capi.MODE_SCALAR, initial_capacity=int(n * 6))
    t = group.tables[0]
    torch.cuda.synchronize()
    kp, vp, op = dk.data_ptr(), dv.data_ptr(), out.data_ptr()

    def step():
        t.push_raw(kp, n, vp, n)
        t.pull_raw(kp, n, op, n)

    for _ in range(max(args.warmup, 3)):  # insert, record, first request served from the cache
        step()
    t.sync()
    t.prof_reset()
    t0 = time.perf_counter()
    for i in range(args.steps):
        t.prof_enable(sampled(i, args.steps))
        step()
    t.sync()
    dt = time.perf_counter() - t0
    push = kernel_stats([t], capi.KERNEL_PUSH_SCALAR)
    pull = kernel_stats([t], capi.KERNEL_PULL_SCALAR)
    same = kernel_stats([t], capi.KERNEL_SAME_KEYS)
    t.prof_enable(False)
    # closed form: every key holds (warm-up + timed steps) sequential adds of its value
    idx = torch.randint(0, n, (4096,), device=dev)
    ref = torch.zeros(4096, device=dev)
    for _ in range(max(args.warmup, 3) + args.steps):
        ref = ref + dv[idx]
    assert torch.equal(out[idx], ref), "sums differ from sequential float adds"
    assert t.size()[0] == n
    # the same step as ONE request with both halves (KVWorker::PushPull, meta.push && meta.pull)
    for _ in range(2):
        t.pushpull_raw(kp, n, vp, n, op, n)
    t.sync()
    t1 = time.perf_counter()
    for _ in range(args.steps):
        t.pushpull_raw(kp, n, vp, n, op, n)
    t.sync()
    dt_pp = time.perf_counter() - t1
    for _ in range(2 + args.steps):
        ref = ref + dv[idx]
    assert torch.equal(out[idx], ref), "push+pull sums differ from sequential float adds"
    # the same step recorded once (pskv_replay_record) and replayed: one call and one launch per step
    whole = np.array([0, n], np.uint64)
    replayed, ref = replay_both(capi, group, args.steps, ref, dv[idx], dk, whole, dv, whole, None, out)
    assert torch.equal(out[idx], ref), "replayed sums differ from sequential float adds"
    res = {
        "value": 2.0 * n * args.steps / dt, "unit": "keys/s", "ms_per_step": dt / args.steps * 1e3,
        "dtype": "f32",
        "replayed": dict(with_rates(replayed, n),
                         one_request={"ms_per_step": dt_pp / args.steps * 1e3, "value": 2.0 * n * args.steps / dt_pp,
                                      "unit": "keys/s",
                                      "note": "the step as one pskv_pushpull request, not recorded: what a recorded "
                                              "SCALAR push + pull is replayed as"}),
        "config": {"workload": "sparse_repeat: the same 16M sorted unique uint64 keys pushed (fresh values) "
                               "and pulled every step, one table", "keys_per_step": n, "ranges": 1,
                   "value_len": 1, "key_dtype": "u64"},
        # 4 val in + 4 cached value read + 4 written; the keys are compared by the kernel in front
        "roofline": dict(roofline(12.0 * n, push[0], push[1], traffic("push_scalar_cached", n), push[2]),
                         kernel="k_scalar<push, cached key set> (cached[i] += v[i])", bytes_per_key=12),
        "kernels": {"pull_scalar_cached": dict(roofline(8.0 * n, pull[0], pull[1],
                                                        traffic("pull_scalar_cached", n), pull[2]),
                                               bytes_per_key=8),
                    "same_keys": dict(roofline(16.0 * n, same[0], same[1], traffic("same_keys", n), same[2]),
                                      kernel="k_same_keys (request keys against cached keys), once per "
                                             "push and once per pull", bytes_per_key=16)},
    }
    return res, (keys, vals, n)


def cpu_sparse_repeat(orc, keys, vals, n, budget_s=20.0):
    store = orc.Store(orc.MODE_SCALAR)
    store.push(keys, vals)  # the inserting first push is not part of the GPU's timed steps either
    done = 0
    t0 = time.perf_counter()
    while done < 1 or time.perf_counter() - t0 < budget_s:
        store.push(keys, vals)
        store.handle(False, True, keys, out_cap=n)
        done += 1
    dt = time.perf_counter() - t0
    return {"value": 2.0 * n * done / dt, "unit": "keys/s", "cores": 1, "kind": "port",
            "sample": "%d steps (push + pull of the same %d keys) on a std::unordered_map store that holds "
                      "them already, one thread" % (done, n)}


# ------------------------------------------------------------------------------------
# embed: rows of an embedding table, other rows in every batch (fixed-length values, kv_app.h:17-22)
# ------------------------------------------------------------------------------------
def run_embed(args, capi, dev):
    """One FIXED table of 8M rows of 64 floats. A step is what a worker does per batch: pull the rows of
    1M keys (another random subset every step), then push a gradient for the same keys. The pull has to
    look its keys up (its comparison with the cached keys would fail, and is soon skipped); the push
    repeats the pull's keys and reuses their row references."""
    import torch
    n, rows, k = args.keys or 1000000, 8000000, 64
    rng = np.random.default_rng(0xE3BED)
    all_keys = unique_sorted_keys(rng, rows, KMAX)
    t = capi.Table(capi.MODE_FIXED, initial_capacity=2 * rows, row_len=k, arena_floats=rows * k + (1 << 20))
    init = torch.ones(rows // 8 * k, dtype=torch.float32, device=dev)
    for c in range(8):  # fill the table: row i starts as all ones
        chunk = to_dev(np.ascontiguousarray(all_keys[c * (rows // 8):(c + 1) * (rows // 8)]), dev)
        t.push(chunk, init)
        t.sync()  # (the call is asynchronous: its buffers stay untouched until the table has used them)
    del init, chunk
    total = args.warmup + args.steps
    batches = []
    for s_ in range(total):
        keys = np.sort(rng.choice(all_keys, size=n, replace=False))
        batches.append(keys)
    d_keys = [to_dev(kk, dev) for kk in batches]
    grad = to_dev(rng.integers(-4, 4, size=n * k).astype(np.float32), dev)  # the same gradient values every step
    out = torch.empty(n * k, dtype=torch.float32, device=dev)
    torch.cuda.synchronize()

    def step(i):
        kp = d_keys[i].data_ptr()
        t.pull_raw(kp, n, out.data_ptr(), n * k)
        t.push_raw(kp, n, grad.data_ptr(), n * k)

    for i in range(args.warmup):
        step(i)
    t.sync()
    t.prof_reset()
    t0 = time.perf_counter()
    for i in range(args.warmup, total):
        t.prof_enable(sampled(i - args.warmup, args.steps))
        step(i)
    t.sync()
    dt = time.perf_counter() - t0
    t.prof_enable(False)
    acc = kernel_stats([t], capi.KERNEL_ROWS_ACC)
    gat = kernel_stats([t], capi.KERNEL_ROWS_GATHER)
    look = kernel_stats([t], capi.KERNEL_LOOKUP)
    # the last pull answered the rows as they were before the last push: ones plus, for every
    # earlier step that named the row, the gradient at the row's place in that step's batch
    # (small integers: exact)
    sample = rng.choice(n, size=2048, replace=False)
    g = grad.cpu().numpy().reshape(n, k)
    keys_s = batches[-1][sample]
    want = np.ones((sample.size, k), np.float32)
    for kk in batches[:-1]:
        at = np.minimum(np.searchsorted(kk, keys_s), n - 1)
        hit = kk[at] == keys_s
        want[hit] += g[at[hit]]
    got = out.cpu().numpy().reshape(n, k)[sample]
    assert np.array_equal(got, want.astype(np.float32)), "pulled rows differ"
    assert t.size()[0] == rows
    res = {
        "value": 2.0 * n * args.steps / dt, "unit": "keys/s", "ms_per_step": dt / args.steps * 1e3,
        "dtype": "f32",
        "config": {"workload": "embed: one table of 8M rows of 64 floats; a step pulls the rows of 1M keys "
                               "(another random subset every step) and pushes a gradient for the same keys",
                   "keys_per_step": n, "ranges": 1, "value_len": k, "key_dtype": "u64",
                   "store_keys_after_timed_steps": rows},
        "gbps": (12.0 + 8.0) * n * k * args.steps / dt / 1e9,
        # gradient in, row in, row out: 12 B/float, the rows scattered over the arena
        "roofline": dict(roofline(12.0 * n * k, acc[0], acc[1], traffic("rows_acc_embed", n * k), acc[2]),
                         kernel="k_rows<acc,fixed> (row += in, rows scattered)", bytes_per_float=12),
        "kernels": {"rows_gather": dict(roofline(8.0 * n * k, gat[0], gat[1],
                                                 traffic("rows_gather_embed", n * k), gat[2]),
                                        bytes_per_float=8),
                    "lookup": dict(roofline(24.0 * n, look[0], look[1], traffic("lookup_embed", n), look[2]),
                                   kernel="k_lookup_fixed (key -> row, the pull's; the push reuses it)",
                                   bytes_per_key=24)},
    }
    return res, (all_keys, batches[args.warmup:], g.reshape(-1), n, rows, k)


def cpu_embed(orc, all_keys, batches, grad, n, rows, k, budget_s=20.0):
    store = orc.Store(orc.MODE_FIXED)
    ones = np.ones(rows // 8 * k, np.float32)
    for c in range(8):
        store.push(all_keys[c * (rows // 8):(c + 1) * (rows // 8)], ones)
    done = 0
    t0 = time.perf_counter()
    for keys in batches:
        store.handle(False, True, keys, out_cap=n * k)
        store.push(keys, grad)
        done += 1
        if time.perf_counter() - t0 > budget_s:
            break
    dt = time.perf_counter() - t0
    return {"value": 2.0 * n * done / dt, "unit": "keys/s", "cores": 1, "kind": "port",
            "sample": "first %d of the timed steps (pull + push of %d rows of %d floats) on a "
                      "std::unordered_map of rows that holds the %d keys already, one thread" % (done, n, k, rows)}


# ------------------------------------------------------------------------------------
# match: the ordered match of two sorted key sets (parallel_kv_match.h:29-120), worker side
# ------------------------------------------------------------------------------------
def run_match(args, capi, dev):
    """A worker merges pulled values into its sorted local parameters: 16M destination keys, 12M source
    keys of which 8M are among the destination's, one float per key, `dst[i] += src[j]` where the keys
    are equal. A step is one pskv_match call (it returns when the destination is complete)."""
    import torch
    n_dst = args.keys or 16000000
    n_src, shared = n_dst * 3 // 4, n_dst // 2
    rng = np.random.default_rng(0xA7C4)
    pool = unique_sorted_keys(rng, n_dst + n_src - shared, KMAX)
    perm = rng.permutation(pool.size)
    src_keys = np.sort(pool[perm[:n_src]])
    dst_keys = np.sort(pool[perm[n_src - shared:]])
    src_vals = rng.integers(-8, 8, size=n_src).astype(np.float32)
    dst_vals = rng.integers(-8, 8, size=n_dst).astype(np.float32)
    d_sk, d_sv, d_dk, d_dv = (to_dev(x, dev) for x in (src_keys, src_vals, dst_keys, dst_vals))
    torch.cuda.synchronize()
    ms = np.zeros(2, np.float32)
    for _ in range(args.warmup):
        capi.match(d_sk, d_sv, d_dk, d_dv, 1, capi.OP_PLUS)
    samples = []
    t0 = time.perf_counter()
    for i in range(args.steps):
        if sampled(i, args.steps):
            matched = capi.match(d_sk, d_sv, d_dk, d_dv, 1, capi.OP_PLUS, kernel_ms=ms)
            samples.append(float(ms[0]))
        else:
            matched = capi.match(d_sk, d_sv, d_dk, d_dv, 1, capi.OP_PLUS)
    dt = time.perf_counter() - t0
    assert matched == shared, (matched, shared)
    # closed form: every shared key holds its value plus (warm-up + timed steps) times the source's
    # (small integers: exact), every other key its own value
    j = np.searchsorted(src_keys, dst_keys)
    hit = (j < n_src) & (src_keys[np.minimum(j, n_src - 1)] == dst_keys)
    want = dst_vals.copy()
    want[hit] += np.float32(args.warmup + args.steps) * src_vals[j[hit]]
    assert np.array_equal(d_dv.cpu().numpy().view(np.uint32), want.view(np.uint32)), "merged values differ"
    # both key sets once, and per matched key the source value in, the destination value in and out
    alg = 8.0 * (n_src + n_dst) + 12.0 * shared
    samples = np.array(samples, np.float32)
    # the same kernel when both sides hold the same keys (a worker that pulled all of its keys):
    # every value line is used in full
    own = torch.zeros(n_dst, dtype=torch.float32, device=dev)
    equal_ms = []
    for i in range(6):
        assert capi.match(d_dk, d_dv, d_dk, own, 1, capi.OP_ASSIGN, kernel_ms=ms) == n_dst
        if i:
            equal_ms.append(float(ms[0]))
    assert torch.equal(own, d_dv)
    equal_ms = np.array(equal_ms, np.float32)
    res = {
        "metric": "source + destination keys/sec of the ordered match and achieved GB/s (% of HBM peak) on 1 MI355X",
        "value": (n_src + n_dst) * args.steps / dt, "unit": "keys/s", "ms_per_step": dt / args.steps * 1e3,
        "dtype": "f32",
        "config": {"workload": "match: sorted source keys (12M) merged into sorted destination keys (16M, 8M "
                               "shared), dst[i] += src[j] where the keys are equal, one float per key",
                   "dst_keys": n_dst, "src_keys": n_src, "shared_keys": shared, "value_len": 1,
                   "key_dtype": "u64"},
        "roofline": dict(roofline(alg, len(samples), float(samples.sum()), traffic("match_keys", n_src + n_dst),
                                  samples),
                         kernel="k_match_keys<k = 1> (stretch of source keys through LDS, values combined)",
                         bytes_per_key=round(alg / (n_src + n_dst), 2)),
        # 8 B per key of either side, source value in, destination value out (ASSIGN reads no old value)
        "kernels": {"match_equal_key_sets": dict(roofline(24.0 * n_dst, len(equal_ms), float(equal_ms.sum()), None,
                                                          equal_ms),
                                                 kernel="k_match_keys<k = 1>, both sides the same %d keys, "
                                                        "dst[i] = src[i]" % n_dst, bytes_per_key=12)},
    }
    return res, (src_keys, src_vals, dst_keys, dst_vals)


def cpu_match(orc, src_keys, src_vals, dst_keys, dst_vals, budget_s=15.0):
    done = 0
    dv = dst_vals
    t0 = time.perf_counter()
    while done < 1 or time.perf_counter() - t0 < budget_s:
        _, dv, _ = orc.ordered_match(src_keys, src_vals, dst_keys, dv, 1, orc.OP_PLUS)
        done += 1
    dt = time.perf_counter() - t0
    return {"value": (src_keys.size + dst_keys.size) * done / dt, "unit": "keys/s", "cores": 1, "kind": "port",
            "sample": "%d calls of the reference's two-pointer loop on the same key sets, one thread (the "
                      "binding copies the destination values once per call)" % done}


# ------------------------------------------------------------------------------------
# Side measurements of the default run: the other BASELINE configurations, each with the CPU
# oracle on the same inputs beside it
# ------------------------------------------------------------------------------------
def extra_plumbing(capi, orc, reps=5):
    """configs[0], the shape of the reference's own test (tests/test_kv_app.cc:27-60) through the
    calls a ps-lite worker and server make: 1,000 keys kMaxKey/1000*i with values 1.0, one server
    range; 50 times slice + push, then slice + pull, everything from and to ordinary host memory
    (PSKV_MEM_HOST). Wall time per request (a request = its slice and its handle call), the
    oracle's slicer and handle on the same arrays beside it."""
    num, S, pushes = 1000, 1, 50
    keys = np.uint64(KMAX // num) * np.arange(num, dtype=np.uint64)
    vals = np.ones(num, np.float32)
    out = np.zeros(num, np.float32)
    rb, re = capi.server_ranges(S)
    walls = []
    for rep in range(reps + 1):  # the first run loads the GPU code and is not counted
        t = capi.Table(capi.MODE_SCALAR)
        t0 = time.perf_counter()
        for _ in range(pushes):
            capi.slice_keys(keys, rb, re, nvals=num)
            t.push(keys, vals)
        capi.slice_keys(keys, rb, re, nvals=0)
        t.pull(keys, out)
        walls.append(time.perf_counter() - t0)
        assert np.all(out == np.float32(pushes)), "pull differs from 50 * v"
        t.close()
    walls = np.array(walls[1:])
    orb, ore = orc.server_ranges(S)
    cpu_walls = []
    for rep in range(reps):
        st = orc.Store(orc.MODE_SCALAR)
        t0 = time.perf_counter()
        for _ in range(pushes):
            orc.slice_keys(keys, orb, ore, nvals=num)
            st.push(keys, vals)
        orc.slice_keys(keys, orb, ore, nvals=0)
        got = st.handle(False, True, keys, out_cap=num)
        cpu_walls.append(time.perf_counter() - t0)
    cpu_walls = np.array(cpu_walls)
    return {"workload": "plumbing: 1,000 keys, 50 x (slice + push) then slice + pull, one key range, host "
                        "buffers through pskv_slice / pskv_push / pskv_pull (PSKV_MEM_HOST)",
            "requests": pushes + 1, "wall_ms": round(float(np.median(walls)) * 1e3, 3),
            "us_per_request": round(float(np.median(walls)) / (pushes + 1) * 1e6, 2),
            "min_us_per_request": round(float(walls.min()) / (pushes + 1) * 1e6, 2),
            "keys_per_s": num * (pushes + 1) / float(np.median(walls)),
            "cpu_baseline": {"us_per_request": round(float(np.median(cpu_walls)) / (pushes + 1) * 1e6, 2),
                             "keys_per_s": num * (pushes + 1) / float(np.median(cpu_walls)), "cores": 1,
                             "kind": "port", "sample": "the same 51 requests through the oracle's slicer and "
                                                       "std::unordered_map handle (ctypes calls included on "
                                                       "both sides), median of %d runs" % reps}}


def extra_replay_small(capi, dev, n=100000, S=4, steps=200):
    """A step whose kernels are short, where the host side decides: the same 100,000 keys over 4 key
    ranges, slice + pskv_push_multi + pskv_pull_multi per step against one pskv_replay_run per step.
    The sums are checked against their closed form both ways."""
    import torch
    rng = np.random.default_rng(0x4E9)
    keys = unique_sorted_keys(rng, n, (KMAX // S) * S)
    dk = to_dev(keys, dev)
    dv = torch.randn(n, device=dev) * 0.01
    out = torch.empty(n, dtype=torch.float32, device=dev)
    rb, re = capi.server_ranges(S)
    group = capi.Group(S, capi.MODE_SCALAR, initial_capacity=n)
    torch.cuda.synchronize()
    kp, vp, op = dk.data_ptr(), dv.data_ptr(), out.data_ptr()

    def step():
        pos, _, _ = capi.slice_keys(dk, rb, re, nvals=n)
        group.push_raw(kp, pos, vp, pos)
        group.pull_raw(kp, pos, op)

    for _ in range(5):
        step()
    group.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    group.sync()
    dt = time.perf_counter() - t0
    ref = torch.zeros(n, device=dev)
    for _ in range(5 + steps):
        ref = ref + dv
    assert torch.equal(out, ref), "sums differ from sequential float adds"

    def step_one():
        pos, _, _ = capi.slice_keys(dk, rb, re, nvals=n)
        group.pushpull_raw(kp, pos, vp, pos, op)

    for _ in range(5):
        step_one()
    group.sync()
    t1 = time.perf_counter()
    for _ in range(steps):
        step_one()
    group.sync()
    dt_one = time.perf_counter() - t1
    for _ in range(5 + steps):
        ref = ref + dv
    assert torch.equal(out, ref), "push+pull sums differ from sequential float adds"
    pos, _, _ = capi.slice_keys(dk, rb, re, nvals=n)
    replayed, ref = replay_both(capi, group, steps, ref, dv, dk, pos, dv, pos, None, out)
    assert torch.equal(out, ref), "replayed sums differ from sequential float adds"
    group.close()
    return {"workload": "the same %d keys over %d key ranges pushed and pulled every step (SCALAR)" % (n, S),
            "steps": steps, "ms_per_step": dt / steps * 1e3, "value": 2.0 * n * steps / dt, "unit": "keys/s",
            "one_request": {"ms_per_step": dt_one / steps * 1e3, "value": 2.0 * n * steps / dt_one, "unit": "keys/s",
                            "note": "slice + ONE pskv_pushpull_multi request per step, not recorded"},
            "replayed": with_rates(replayed, n)}


def extra_host_staged(capi, reps=2, nk=64, k=4194304):
    """configs[2] from and to ordinary (pageable) host memory, as a server gets it from the
    transport: 1 GiB per push and per pull through PSKV_MEM_HOST. PCIe-inclusive, never `value`."""
    keys = np.uint64(KMAX // nk) * np.arange(nk, dtype=np.uint64)
    vals = np.full(nk * k, 0.5, np.float32)
    out = np.empty(nk * k, np.float32)
    out[::1024] = 0  # (touch the pages)
    t = capi.Table(capi.MODE_FIXED, initial_capacity=1024, row_len=k, arena_floats=nk * k)
    t.push(keys, vals)  # creates the rows; also warms the staging ring
    push_s, pull_s = [], []
    for _ in range(reps):
        t0 = time.perf_counter()
        t.push(keys, vals)
        t1 = time.perf_counter()
        t.pull(keys, out)
        t2 = time.perf_counter()
        push_s.append(t1 - t0)
        pull_s.append(t2 - t1)
    assert out[12345] == np.float32(0.5 * (reps + 1)) and out[-1] == np.float32(0.5 * (reps + 1))
    t.close()
    gib = nk * k * 4 / 1e9
    return {"workload": "dense from host memory: 64 keys x 4,194,304 f32 (1 GiB) pushed from and pulled "
                        "into ordinary host memory, PCIe-inclusive",
            "push_gb_per_s": round(gib / min(push_s), 2), "pull_gb_per_s": round(gib / min(pull_s), 2),
            "push_ms": round(min(push_s) * 1e3, 2), "pull_ms": round(min(pull_s) * 1e3, 2),
            "note": "best of %d; inside this Python process the HIP runtime that torch brings serves the "
                    "library, whose device-to-pinned copies block the calling thread: a C++ server gets "
                    "about twice this pull rate" % reps}


def brief(res, cpu=None):
    """What an `extra` entry keeps of a workload's result."""
    out = {k: res[k] for k in ("value", "unit", "ms_per_step", "gbps", "phases", "replayed") if k in res}
    out["workload"] = res["config"]["workload"]
    out["roofline"] = res["roofline"]
    out["kernels"] = res.get("kernels")
    if cpu is not None:
        out["cpu_baseline"] = cpu
    return out


def main():
    global SAMPLE_EVERY
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="sparse_lr", choices=["sparse_lr", "dense", "varlen", "zipf", "sparse_repeat", "embed", "match"])
    ap.add_argument("--keys", type=int, default=0, help="keys per step (default: the config's)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the dense-chunk side measurement")
    ap.add_argument("--no-rehearsal", action="store_true",
                    help="sparse_lr: measure the first run of the process (no untimed run on tables of its own first)")
    ap.add_argument("--sample-every", type=int, default=SAMPLE_EVERY,
                    help="every how many timed steps the launches carry events of their own")
    ap.add_argument("--per-table", action="store_true",
                    help="sparse_lr / varlen: serve the key ranges with one pskv_push / pskv_pull per table "
                         "instead of one pskv_push_multi / pskv_pull_multi over all of them")
    ap.add_argument("--own-streams", action="store_true",
                    help="sparse_lr / varlen: also time the steps with one stream per table "
                         "(reported under extra.own_streams; kernels of different ranges overlap)")
    args = ap.parse_args()
    SAMPLE_EVERY = max(1, args.sample_every)
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures ONE GPU: a table lives on one device and nothing here uses a "
              "second one; run it with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    dev = torch.device("cuda:0")
    capi = graft.load_package().capi
    capi.load()  # raises if libpskv.so is missing: there is no other path
    wake_gpu(dev)

    if args.workload == "sparse_lr":
        res, timed_batches, (n, S) = run_sparse_lr(args, capi, dev)
    elif args.workload == "dense":
        res = run_dense(args, capi, dev)
    elif args.workload == "zipf":
        args.steps = 8  # the configuration is 8 worker pushes and a pull
        res, zipf_inputs = run_zipf(args, capi, dev)
    elif args.workload == "sparse_repeat":
        res, repeat_inputs = run_sparse_repeat(args, capi, dev)
    elif args.workload == "match":
        res, match_inputs = run_match(args, capi, dev)
    elif args.workload == "embed":
        res, embed_inputs = run_embed(args, capi, dev)
    else:
        res, varlen_inputs = run_varlen(args, capi, dev)

    extra = {}
    orc = None if args.no_cpu else graft.load_oracle()
    if args.workload == "sparse_lr" and not args.no_extra:
        # the dense-chunk kernels carry the bandwidth target of this path; measure them
        # beside the default workload (12 push+pull steps of 1 GiB, every launch timed)
        dt, acc, gat, cp, nk, k = measure_dense(capi, dev, 12, 2, every_step=True)
        extra["dense_chunk"] = {
            "workload": "dense: 64 keys x 4,194,304 f32 (1 GiB), push-accumulate then full pull, 12 steps",
            "value": 20.0 * nk * k * 12 / dt / 1e9, "unit": "GB/s", "ms_per_step": dt / 12 * 1e3,
            "rows_acc": dict(roofline(12.0 * nk * k, acc[0], acc[1], traffic("rows_acc_fixed", nk * k), acc[2]),
                             bytes_per_float=12),
            "rows_gather": dict(roofline(8.0 * nk * k, gat[0], gat[1],
                                         traffic("rows_gather_fixed", nk * k), gat[2]), bytes_per_float=8),
            "copy_ceiling": dict(roofline(8.0 * nk * k, cp[0], cp[1], 8.0 * nk * k, cp[2]),
                                 kernel="k_copy (plain copy of 1 GiB)"),
        }
        if orc is not None:
            extra["dense_chunk"]["cpu_baseline"] = cpu_dense(orc, budget_s=3.0)
        extra["host_staged"] = extra_host_staged(capi)
        sub = argparse.Namespace(**vars(args))
        sub.steps, sub.warmup, sub.keys, sub.per_table, sub.own_streams = 10, 2, 0, False, False
        log("extra: varlen")
        vres, vin = run_varlen(sub, capi, dev)
        extra["varlen"] = brief(vres, cpu_varlen(orc, *vin, budget_s=4.0) if orc is not None else None)
        del vin
        log("extra: zipf")
        zres, zin = run_zipf(sub, capi, dev)
        extra["zipf"] = brief(zres, cpu_zipf(orc, *zin, budget_s=12.0) if orc is not None else None)
        del zin
        if orc is not None:
            log("extra: plumbing")
            extra["plumbing"] = extra_plumbing(capi, orc)
        # stable key sets (the same keys every step) and the ordered match of two sorted key sets
        log("extra: sparse_repeat")
        sub.steps, sub.warmup = 10, 3
        rres, rin = run_sparse_repeat(sub, capi, dev)
        extra["sparse_repeat"] = brief(rres, cpu_sparse_repeat(orc, *rin, budget_s=3.0) if orc is not None else None)
        del rin
        extra["replay_small"] = extra_replay_small(capi, dev)
        log("extra: embed")
        eres, ein = run_embed(sub, capi, dev)
        extra["embed"] = brief(eres, cpu_embed(orc, *ein, budget_s=3.0) if orc is not None else None)
        del ein
        log("extra: match")
        mres, min_ = run_match(sub, capi, dev)
        extra["match"] = brief(mres, cpu_match(orc, *min_, budget_s=3.0) if orc is not None else None)
        del min_

    cpu = None
    if not args.no_cpu:
        log("timing the CPU oracle (bounded sample)")
        if args.workload == "sparse_lr":
            cpu = cpu_sparse_lr(orc, timed_batches, n, S)
        elif args.workload == "dense":
            cpu = cpu_dense(orc)
            extra["cpu_baseline_all_cores"] = cpu_dense_all_cores(orc)
        elif args.workload == "zipf":
            cpu = cpu_zipf(orc, *zipf_inputs)
        elif args.workload == "sparse_repeat":
            cpu = cpu_sparse_repeat(orc, *repeat_inputs)
        elif args.workload == "match":
            cpu = cpu_match(orc, *match_inputs)
        elif args.workload == "embed":
            cpu = cpu_embed(orc, *embed_inputs)
        else:
            cpu = cpu_varlen(orc, *varlen_inputs)
        cpu["host"] = host_info()

    line = {
        "metric": res.get("metric", "push+pull keys/sec and achieved GB/s (% of HBM peak) on 1 MI355X"),
        "value": res["value"], "unit": res["unit"], "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": res["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": res["dtype"], "data": "synthetic",
        "config": res["config"], "roofline": res["roofline"], "cpu_baseline": cpu,
        "kernels": res.get("kernels"),
    }
    line["roofline"]["traffic_source"] = (
        "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE per dispatch of this command, scaled by the 1 GiB copy "
        "kernel; read at run time from " + ", ".join(sorted(TRAFFIC_SOURCES))) if TRAFFIC_SOURCES else None
    if "gbps" in res:
        line["gbps"] = res["gbps"]
    for k in ("own_streams", "presized", "per_table", "multi", "replayed"):
        if k in res:
            extra[k] = res[k]
    if "phases" in res:
        line["phases"] = res["phases"]
    if extra:
        line["extra"] = extra
    print(json.dumps(line, allow_nan=False), flush=True)  # strict JSON: a NaN would be a bug


if __name__ == "__main__":
    main()
