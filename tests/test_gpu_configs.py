"""The five BASELINE configurations at their full sizes on the GPU, bit-exact against the CPU
oracle on the same seeded inputs (each oracle leg finishes in seconds), plus size-independent
properties: exact integer sums, stored-key sets, idempotent pulls, slice/reassembly round trips."""
import numpy as np
import pytest

from conftest import announce
from helpers import KMAX, assert_bits_equal, covered_limit, from_dev, to_dev, unique_keys

pytestmark = pytest.mark.gpu


def _slices(capi, dk, rb, re, dl=None, nvals=0):
    pos, vpos, used = capi.slice_keys(dk, rb, re, lens=dl, nvals=nvals)
    return [int(x) for x in pos], [int(x) for x in vpos], used


def test_config1_plumbing_shape(capi, orc, dev):
    """1,000 keys spread evenly over the key range, all 1.0, 50 pushes then a pull, one server."""
    import torch
    announce("config1")
    n = 1000
    keys = np.uint64(KMAX // n) * np.arange(n, dtype=np.uint64)
    vals = np.ones(n, np.float32)
    rb, re = capi.server_ranges(1)
    dk, dv = to_dev(keys, dev), to_dev(vals, dev)
    t = capi.Table(capi.MODE_SCALAR)
    o = orc.Store(orc.MODE_SCALAR)
    for _ in range(50):
        pos, _, used = _slices(capi, dk, rb, re, nvals=n)
        assert pos == [0, n] and used[0] == 1
        t.push(dk, dv)
        o.push(keys, vals)
    out = torch.zeros(n, dtype=torch.float32, device=dev)
    t.pull(dk, out)
    t.sync()
    assert np.all(from_dev(out) == np.float32(50.0))
    assert_bits_equal(from_dev(out), o.pull(keys)[0], "config1")


def test_config2_sparse_lr_full(capi, orc, dev):
    """20 pushes of 1M fresh uniform keys over 4 ranges (store grows to 20M), then pulls."""
    import torch
    announce("config2 full size")
    n, S, pushes = 1000000, 4, 20
    rb, re = capi.server_ranges(S)
    tables = [capi.Table(capi.MODE_SCALAR, initial_capacity=1 << 20) for _ in range(S)]  # grows 3 times
    stores = [orc.Store(orc.MODE_SCALAR) for _ in range(S)]
    all_keys = []
    for p in range(pushes):
        rng = np.random.default_rng(0xC0FFEE + p)
        keys = unique_keys(rng, n, S)
        vals = rng.normal(0, 0.01, size=n).astype(np.float32)
        all_keys.append(keys)
        dk, dv = to_dev(keys, dev), to_dev(vals, dev)
        pos, _, used = _slices(capi, dk, rb, re, nvals=n)
        o_pos, _, o_used = orc.slice_keys(keys, rb, re, nvals=n)
        assert pos == [int(x) for x in o_pos] and np.array_equal(used, o_used)
        for s in range(S):
            tables[s].push(dk[pos[s]:pos[s + 1]], dv[pos[s]:pos[s + 1]])
            stores[s].push(keys[pos[s]:pos[s + 1]], vals[pos[s]:pos[s + 1]])
        for t in tables:
            t.sync()  # dk/dv are released after this iteration
    # pull of the last push's keys, then of a mix of old keys and absent keys (which get created)
    rng = np.random.default_rng(5)
    mix = np.unique(np.concatenate([rng.choice(np.concatenate(all_keys[:5]), size=500000, replace=False),
                                    unique_keys(rng, 200000, S)]))
    for probe in (all_keys[-1], mix):
        dk = to_dev(probe, dev)
        out = torch.empty(probe.size, dtype=torch.float32, device=dev)
        pos, _, used = _slices(capi, dk, rb, re, nvals=0)
        want = np.empty(probe.size, np.float32)
        for s in range(S):
            tables[s].pull(dk[pos[s]:pos[s + 1]], out[pos[s]:pos[s + 1]])
            want[pos[s]:pos[s + 1]] = stores[s].pull(probe[pos[s]:pos[s + 1]])[0]
        for t in tables:
            t.sync()
        assert_bits_equal(from_dev(out), want, "config2 pull")
    for s in range(S):
        assert tables[s].size() == stores[s].size()
    gk, _, gv = tables[1].dump()
    ok, _, ov = stores[1].dump()
    assert np.array_equal(gk, ok)
    assert_bits_equal(gv, ov, "config2 dump of range 1")


def test_config3_dense_chunks_full(capi, orc, dev):
    """64 keys x 4,194,304 f32 (1 GiB per push), 8 worker pushes in fixed order, one full pull."""
    import torch
    announce("config3 full size")
    nk, k, workers = 64, 4194304, 8
    keys = np.uint64(KMAX // nk) * np.arange(nk, dtype=np.uint64)
    dk = to_dev(keys, dev)
    t = capi.Table(capi.MODE_FIXED, row_len=k, arena_floats=nk * k)
    o = orc.Store(orc.MODE_FIXED, k)
    for w in range(workers):
        vals = np.random.default_rng(0xD15E + w).uniform(-1, 1, size=nk * k).astype(np.float32)
        dv = to_dev(vals, dev)
        t.push(dk, dv)
        o.push(keys, vals)
        t.sync()
        del dv
    out = torch.empty(nk * k, dtype=torch.float32, device=dev)
    assert t.pull(dk, out) == nk * k
    t.sync()
    want = np.empty(nk * k, np.float32)
    rc, want, _, _ = o.handle(False, True, keys, out_cap=nk * k)
    assert rc == 0
    assert_bits_equal(from_dev(out), want, "config3")
    assert t.size() == (nk, nk * k)


def test_config3_dense_chunks_from_host_memory(capi, orc, dev):
    """Configuration 3 the way a ps-lite server gets it: the 1 GiB of every push sits in ordinary host
    memory and the pull answers into host memory. 3 worker pushes and a full pull, bit for bit against
    the oracle; the requests travel through the ring of pinned pieces, 128 pieces per GiB."""
    import time
    announce("config3 from host memory")
    nk, k, workers = 64, 4194304, 3
    keys = np.uint64(KMAX // nk) * np.arange(nk, dtype=np.uint64)
    t = capi.Table(capi.MODE_FIXED, row_len=k, arena_floats=nk * k)
    o = orc.Store(orc.MODE_FIXED, k)
    secs = []
    for w in range(workers):
        vals = np.random.default_rng(0xD15E + w).uniform(-1, 1, size=nk * k).astype(np.float32)
        t0 = time.perf_counter()
        t.push(keys, vals)
        secs.append(time.perf_counter() - t0)
        o.push(keys, vals)
    out = np.empty(nk * k, np.float32)
    t0 = time.perf_counter()
    assert t.pull(keys, out) == nk * k
    pull_s = time.perf_counter() - t0
    rc, want, _, _ = o.handle(False, True, keys, out_cap=nk * k)
    assert rc == 0
    assert_bits_equal(out, want, "config3 host")
    print("host-resident 1 GiB push: %s GB/s, pull: %.1f GB/s" % (
        ", ".join("%.1f" % (nk * k * 4 / s / 1e9) for s in secs), nk * k * 4 / pull_s / 1e9))


def test_config2_as_the_benchmark_runs_it(capi, orc, dev):
    """The measured path itself at full size: four tables of the default capacity that share one
    stream, every step one pskv_slice, ONE pskv_push_multi over the four key ranges and ONE
    pskv_pull_multi of the same keys (served from what the push left behind once the tables have
    seen a pull follow a push), no wait inside the run, the tables growing as they go. EVERY
    step's pull is compared with the oracle's, then the four sizes and the dump of one table."""
    import torch
    announce("config2 as benched")
    n, S, steps = 1000000, 4, 20
    rb, re = capi.server_ranges(S)
    group = capi.Group(S, capi.MODE_SCALAR)
    stores = [orc.Store(orc.MODE_SCALAR) for _ in range(S)]
    batches = []
    for p in range(steps):
        rng = np.random.default_rng(0xC0FFEE + p)
        keys = unique_keys(rng, n, S)
        batches.append((keys, rng.normal(0, 0.01, size=n).astype(np.float32)))
    # three steps repeat earlier key sets, so that pushes also meet keys that are stored already
    batches[7] = (batches[2][0], batches[7][1])
    batches[13] = (batches[12][0], batches[13][1])
    batches[19] = (batches[12][0], batches[19][1])
    d_batches = [(to_dev(k, dev), to_dev(v, dev)) for k, v in batches]
    outs = [torch.full((n,), 7.0, dtype=torch.float32, device=dev) for _ in range(steps)]
    torch.cuda.synchronize()
    for p in range(steps):
        dk, dv = d_batches[p]
        pos, vpos, used = capi.slice_keys(dk, rb, re, nvals=n)
        group.push_raw(dk.data_ptr(), pos, dv.data_ptr(), vpos)
        group.pull_raw(dk.data_ptr(), pos, outs[p].data_ptr())
    group.sync()
    held = 0
    for p in range(steps):
        keys, vals = batches[p]
        o_pos, _, _ = orc.slice_keys(keys, rb, re, nvals=n)
        o_pos = [int(x) for x in o_pos]
        want = np.empty(n, np.float32)
        for s in range(S):
            a, b = o_pos[s], o_pos[s + 1]
            stores[s].push(keys[a:b], vals[a:b])
            want[a:b] = stores[s].pull(keys[a:b])[0]
        assert_bits_equal(from_dev(outs[p]), want, "pull of step %d" % p)
    for s in range(S):
        c = group.tables[s].counters()
        # every table grew (from 4M slots) without ever waiting for the stream to size itself
        assert c["growths"] >= 1 and c["growths_unasked"] == c["growths"] and c["waits"] == 0, c
        assert group.tables[s].size() == stores[s].size(), s
        held += group.tables[s].size()[0]
    assert held == np.unique(np.concatenate([k for k, _ in batches])).size
    gk, _, gv = group.tables[2].dump()
    ok, _, ov = stores[2].dump()
    assert np.array_equal(gk, ok)
    assert_bits_equal(gv, ov, "dump of table 2")
    group.close()


def _zipf_unique(rng, n, universe, s=1.1):
    """n distinct ranks with Zipf(s) popularity (the benchmark's generator: the set of ranks that
    a long run of draws names, without drawing them one by one)."""
    import bench
    return bench.zipf_distinct_ranks(rng, n, universe, s)


def _rank_to_key(r):
    """An injective scatter of ranks over the covered key space (odd multiplier mod 2^64, then >> 1)."""
    return ((r.astype(np.uint64) * np.uint64(0x9E3779B97F4A7C15)) >> np.uint64(1)).astype(np.uint64)


@pytest.mark.parametrize("scale,model", [(8, "oracle"), (1, "integers"), (1, "oracle")])
def test_config4_zipf(capi, orc, dev, scale, model):
    """8 worker pushes of Zipf(1.1)-popular keys from a 100M-key universe, then a pull of Zipf keys
    of which many are absent. With model "oracle" the values are N(0,1) and everything pulled is
    compared with the oracle float for float: at one eighth of the size (where the whole store is
    dumped and compared as well) and at the full size (4M keys per push, 16M pulled). Model
    "integers" is a second, independent check at full size: small-integer values, whose sums are
    exact in any order, against numpy."""
    import torch
    announce("config4", scale, model)
    universe, n_push, n_pull, workers = 100000000 // scale, 4000000 // scale, 16000000 // scale, 8
    t = capi.Table(capi.MODE_SCALAR, initial_capacity=1 << 20)
    o = orc.Store(orc.MODE_SCALAR) if model == "oracle" else None
    pushed_ranks, pushed_vals = [], []
    for w in range(workers):
        rng = np.random.default_rng(0x21F + w)
        ranks = _zipf_unique(rng, n_push, universe)
        keys = np.sort(_rank_to_key(ranks))
        vals = rng.standard_normal(n_push).astype(np.float32) if o else \
            rng.integers(-500, 500, size=n_push).astype(np.float32)
        assert np.all(np.diff(keys.astype(np.int64 if keys.max() < 2 ** 63 else np.uint64)) != 0)
        t.push(to_dev(keys, dev), to_dev(vals, dev))
        t.sync()
        if o:
            o.push(keys, vals)
        pushed_ranks.append(keys)
        pushed_vals.append(vals)
    rng = np.random.default_rng(0x9011)
    probe = np.sort(_rank_to_key(_zipf_unique(rng, n_pull, universe)))
    dk = to_dev(probe, dev)
    out = torch.empty(probe.size, dtype=torch.float32, device=dev)
    t.pull(dk, out)
    t.sync()
    got = from_dev(out)
    if o:
        assert_bits_equal(got, o.pull(probe)[0], "config4")
        assert t.size() == o.size()
        if scale > 1:
            gk, _, gv = t.dump()
            ok, _, ov = o.dump()
            assert np.array_equal(gk, ok)
            assert_bits_equal(gv, ov, "config4 dump")
        else:
            # every key ever pushed, pulled back: the whole store float for float without the
            # host-side sort of a dump
            everything = np.unique(np.concatenate(pushed_ranks))
            out_all = torch.empty(everything.size, dtype=torch.float32, device=dev)
            t.pull(to_dev(everything, dev), out_all)
            t.sync()
            assert_bits_equal(from_dev(out_all), o.pull(everything)[0], "config4 all pushed keys")
            assert t.size() == o.size()
    else:
        allk = np.concatenate(pushed_ranks)
        allv = np.concatenate(pushed_vals).astype(np.int64)
        order = np.argsort(allk, kind="stable")
        allk, allv = allk[order], allv[order]
        uk, start = np.unique(allk, return_index=True)
        sums = np.add.reduceat(allv, start)
        idx = np.searchsorted(uk, probe)
        idx[idx == uk.size] = 0
        hit = uk[idx] == probe
        want = np.where(hit, sums[idx], 0).astype(np.float32)
        assert np.array_equal(got, want)
        # a pull creates the absent keys: the store now holds the union
        assert t.size()[0] == np.union1d(uk, probe).size
        # pulling again changes nothing
        out2 = torch.empty_like(out)
        t.pull(dk, out2)
        t.sync()
        assert torch.equal(out, out2)


def test_config5_varlen_rows_full(capi, orc, dev):
    """2M keys with lens in {8,16,32,64,128} over 16 ranges, 10 pushes, then a pull with lens."""
    import torch
    announce("config5 full size")
    n, S, pushes = 2000000, 16, 10
    rb, re = capi.server_ranges(S)
    keys = unique_keys(np.random.default_rng(0xE3B), n, S)
    lens = np.random.default_rng(0xE3C).choice(np.array([8, 16, 32, 64, 128], np.int32), size=n).astype(np.int32)
    nvals = int(lens.sum())
    dk, dl = to_dev(keys, dev), to_dev(lens, dev)
    pos, vpos, used = _slices(capi, dk, rb, re, dl, nvals)
    o_pos, o_vpos, o_used = orc.slice_keys(keys, rb, re, lens, nvals)
    assert pos == [int(x) for x in o_pos] and vpos == [int(x) for x in o_vpos]
    tables = [capi.Table(capi.MODE_VARLEN, initial_capacity=n // S) for _ in range(S)]
    o = orc.Store(orc.MODE_VARLEN)  # one oracle store: the ranges are disjoint
    for p in range(pushes):
        vals = np.random.default_rng(0xE3D + p).normal(0, 0.1, size=nvals).astype(np.float32)
        dv = to_dev(vals, dev)
        for s in range(S):
            tables[s].push(dk[pos[s]:pos[s + 1]], dv[vpos[s]:vpos[s + 1]], dl[pos[s]:pos[s + 1]])
        o.push(keys, vals, lens)
        for t in tables:
            t.sync()
    out = torch.empty(nvals, dtype=torch.float32, device=dev)
    out_lens = torch.empty(n, dtype=torch.int32, device=dev)
    responses = []
    for s in range(S):
        ks = dk[pos[s]:pos[s + 1]]
        part = torch.empty(vpos[s + 1] - vpos[s], dtype=torch.float32, device=dev)
        part_lens = torch.empty(ks.numel(), dtype=torch.int32, device=dev)
        assert tables[s].pull(ks, part, part_lens) == part.numel()
        responses.append((ks, part, part_lens))
    for t in tables:
        t.sync()
    assert capi.assemble_pull(dk, responses[::-1], out, out_lens) == nvals
    want, want_lens = o.pull(keys)
    assert np.array_equal(from_dev(out_lens), want_lens)
    assert_bits_equal(from_dev(out), want, "config5")
    assert sum(t.size()[0] for t in tables) == n
    assert sum(t.size()[1] for t in tables) == nvals
