"""GPU parity of the store (request handle) against the CPU oracle, through the C ABI.
Bar: bit-exact pulled values, identical stored key sets, identical sizes."""
import numpy as np
import pytest

from conftest import announce
from helpers import KMAX, assert_bits_equal, from_dev, to_dev, unique_keys

pytestmark = pytest.mark.gpu


def _check_dump(t, o, what):
    gk, gl, gv = t.dump()
    ok, ol, ov = o.dump()
    assert np.array_equal(gk, ok), what + ": stored keys differ"
    assert np.array_equal(gl, ol), what + ": stored lens differ"
    assert_bits_equal(gv, ov, what + " dump")
    assert t.size() == o.size()


@pytest.mark.parametrize("memkind", ["device", "host"])
@pytest.mark.parametrize("n,cap", [(1, 0), (1000, 16), (50000, 1024)])
def test_scalar_push_pull(capi, orc, dev, memkind, n, cap):
    import torch
    announce("scalar_push_pull", memkind, n, cap)
    rng = np.random.default_rng(100 + n)
    t = capi.Table(capi.MODE_SCALAR, initial_capacity=cap)
    o = orc.Store(orc.MODE_SCALAR)
    universe = unique_keys(rng, 2 * n)
    for rep in range(4):
        keys = np.sort(rng.choice(universe, size=n, replace=False))
        vals = rng.standard_normal(n).astype(np.float32)
        if memkind == "device":
            t.push(to_dev(keys, dev), to_dev(vals, dev))
        else:
            t.push(keys, vals)
        o.push(keys, vals)
    keys = np.sort(rng.choice(universe, size=n, replace=False))
    want, _ = o.pull(keys)
    if memkind == "device":
        out = torch.full((n,), 7.0, dtype=torch.float32, device=dev)
        assert t.pull(to_dev(keys, dev), out) == n
        t.sync()
        got = from_dev(out)
    else:
        got = np.full(n, 7.0, np.float32)
        assert t.pull(keys, got) == n
    assert_bits_equal(got, want, "pull")
    _check_dump(t, o, "scalar")


def test_scalar_closed_form_50_pushes(capi, dev):
    """tests/test_kv_app.cc:27-60: keys kMaxKey/num*i, 50 pushes then pull == 50*v, 50 more
    push+pulls == 100*v."""
    import torch
    announce("scalar_closed_form")
    num = 1000
    keys = (np.uint64(KMAX // num) * np.arange(num, dtype=np.uint64))
    vals = np.random.default_rng(7).integers(0, 1000, size=num).astype(np.float32)
    t = capi.Table(capi.MODE_SCALAR)
    dk, dv = to_dev(keys, dev), to_dev(vals, dev)
    for _ in range(50):
        t.push(dk, dv)
    out = torch.zeros(num, dtype=torch.float32, device=dev)
    t.pull(dk, out)
    t.sync()
    assert np.array_equal(from_dev(out), vals * 50)
    for _ in range(50):
        t.pushpull(dk, dv, out)
    t.sync()
    assert np.array_equal(from_dev(out), vals * 100)
    assert t.size() == (num, num)


def test_scalar_special_values(capi, orc, dev):
    """-0.0 on a fresh key stores +0.0 (0.0f + v), denormals are kept, a pull creates absent keys,
    and key 2^64-1 is an ordinary key for the handle."""
    announce("scalar_special_values")
    keys = np.array([0, 1, 5, 77, KMAX - 1, KMAX], np.uint64)
    v1 = np.array([-0.0, 1e-42, np.inf, 3.5, -2.25, 9.0], np.float32)
    v2 = np.array([-0.0, 1e-42, -1.0, 1e-45, 2.25, 1.0], np.float32)
    t = capi.Table(capi.MODE_SCALAR)
    o = orc.Store(orc.MODE_SCALAR)
    for v in (v1, v2):
        t.push(keys, v)
        o.push(keys, v)
    probe = np.array([0, 1, 2, 5, 77, 1000, KMAX - 1, KMAX], np.uint64)
    got = np.full(probe.size, 5.0, np.float32)
    t.pull(probe, got)
    want, _ = o.pull(probe)
    assert_bits_equal(got, want, "special")
    assert got.view(np.uint32)[0] == 0  # +0.0, not 0x80000000
    assert t.size() == o.size() == (8, 8)
    _check_dump(t, o, "special")


def test_scalar_growth(capi, orc, dev):
    """The slot array grows from its minimum to 300k keys; sums survive every rehash."""
    announce("scalar_growth")
    rng = np.random.default_rng(5)
    t = capi.Table(capi.MODE_SCALAR, initial_capacity=1)
    o = orc.Store(orc.MODE_SCALAR)
    universe = unique_keys(rng, 300000)
    for rep in range(6):
        keys = np.sort(universe[rng.random(universe.size) < 0.5])
        vals = rng.standard_normal(keys.size).astype(np.float32)
        t.push(to_dev(keys, dev), to_dev(vals, dev))
        o.push(keys, vals)
    _check_dump(t, o, "growth")


@pytest.mark.parametrize("max_load", [0.25, 0.5, 0.9])
@pytest.mark.parametrize("first,step", [(400, 400), (1000, 1000), (300, 5000), (40000, 9000)])
def test_growth_by_every_factor(capi, orc, dev, max_load, first, step):
    """A growth by 2, 4 or 8 streams the old array into the new one stretch by stretch and hands
    the keys of probe chains that cross a stretch (or wrap around the end of the array, frequent
    at fill 0.9) to a second pass; a growth by more re-inserts every key. Whatever the factor and
    the fill, every key and every sum arrives: the dump equals the oracle's after every push."""
    announce("growth_by_every_factor", max_load, first, step)
    rng = np.random.default_rng(int(max_load * 100) + first)
    t = capi.Table(capi.MODE_SCALAR, initial_capacity=first, max_load=max_load)
    o = orc.Store(orc.MODE_SCALAR)
    universe = unique_keys(rng, 16 * step + first)
    at = 0
    for rep in range(12):
        fresh = universe[at:at + step]
        at += step
        again = universe[:at][rng.random(at) < 0.1]  # some of the keys held already
        keys = np.unique(np.concatenate([fresh, again]))
        vals = rng.integers(-50, 50, size=keys.size).astype(np.float32)
        t.push(to_dev(keys, dev), to_dev(vals, dev))
        o.push(keys, vals)
        if rep % 3 == 2:
            _check_dump(t, o, "after push %d" % rep)
    _check_dump(t, o, "growth")


@pytest.mark.parametrize("max_load,first,second", [(0.5, 1500, 3000), (0.9, 3500, 6000)])
def test_growth_by_eight(capi, orc, dev, max_load, first, second):
    """A request that needs between four and eight times the slots makes the array eight times as
    large in one streaming move (the largest factor that goes that way): 4,096 slots that hold
    `first` keys, at a fill of 0.37 or 0.85 (long probe chains, some wrapped around the end of the
    array), become 32,768."""
    announce("growth_by_eight", max_load)
    rng = np.random.default_rng(int(max_load * 10))
    t = capi.Table(capi.MODE_SCALAR, initial_capacity=2000, max_load=max_load)
    o = orc.Store(orc.MODE_SCALAR)
    universe = unique_keys(rng, first + second)
    perm = rng.permutation(universe.size)
    a, b = np.sort(universe[perm[:first]]), np.sort(universe[perm[first:]])
    for keys in (a, b):
        vals = rng.integers(-50, 50, size=keys.size).astype(np.float32)
        if keys is a:
            assert t.counters()["slots"] == 4096
        t.push(to_dev(keys, dev), to_dev(vals, dev))
        o.push(keys, vals)
    c = t.counters()
    assert c["slots"] == 32768 and c["growths"] == 1 and c["waits"] == 0, c
    _check_dump(t, o, "growth by eight")


def test_growth_of_a_large_array_by_two(capi, orc, dev):
    """Arrays beyond 64 MB double: 4.6M keys take a table through 4x growths and then a 2x one."""
    announce("growth_of_a_large_array")
    rng = np.random.default_rng(77)
    t = capi.Table(capi.MODE_SCALAR)
    o = orc.Store(orc.MODE_SCALAR)
    universe = unique_keys(rng, 4600000)
    for part in np.array_split(universe, 10):
        vals = rng.integers(-50, 50, size=part.size).astype(np.float32)
        t.push(to_dev(part, dev), to_dev(vals, dev))
        o.push(part, vals)
    probe = np.sort(rng.choice(universe, size=200000, replace=False))
    got = np.zeros(probe.size, np.float32)
    t.pull(probe, got)
    assert_bits_equal(got, o.pull(probe)[0], "pull after the growths")
    _check_dump(t, o, "large growth")


def test_device_trim_between_growths(capi, orc, dev):
    """pskv_device_trim gives back what the pool keeps (the arrays that growths have replaced) and the
    workspaces of pskv_match; tables that are alive keep working, grow again and stay exact."""
    import torch
    announce("device_trim")
    rng = np.random.default_rng(808)
    t = capi.Table(capi.MODE_SCALAR, initial_capacity=1000)
    o = orc.Store(orc.MODE_SCALAR)
    universe = unique_keys(rng, 400000)
    for part in np.array_split(universe, 8)[:4]:
        vals = rng.integers(-9, 9, size=part.size).astype(np.float32)
        t.push(to_dev(part, dev), to_dev(vals, dev))
        o.push(part, vals)
    sk = unique_keys(rng, 5000)
    dst = torch.zeros(sk.size, dtype=torch.float32, device=dev)
    assert capi.match(to_dev(sk, dev), to_dev(np.ones(sk.size, np.float32), dev), to_dev(sk, dev), dst, 1, capi.OP_PLUS) == sk.size
    capi.device_trim()   # requests may be in flight: the call waits for the device first
    capi.device_trim()   # nothing left to give back: still fine
    for part in np.array_split(universe, 8)[4:]:
        vals = rng.integers(-9, 9, size=part.size).astype(np.float32)
        t.push(to_dev(part, dev), to_dev(vals, dev))
        o.push(part, vals)
    assert capi.match(to_dev(sk, dev), to_dev(np.ones(sk.size, np.float32), dev), to_dev(sk, dev), dst, 1, capi.OP_PLUS) == sk.size
    assert torch.all(dst == 2.0)
    _check_dump(t, o, "after the trim")
    t.close()
    capi.device_trim()


@pytest.mark.parametrize("mode", ["scalar", "fixed"])
def test_a_table_does_not_grow_for_keys_that_are_not_coming(capi, orc, dev, mode):
    """A table at a fill of 0.33 whose caller keeps many large requests in flight that name keys it
    holds: counted in full, the keys in flight would take the table over its fill limit (0.7M held + two
    requests of 0.2M unaccounted for + the request at hand = 1.3M against 1.05M), so it used to double
    for nothing. The host now counts them with the share that the device's records say is new, and in
    full only against a limit the array must never cross. When the requests then bring new keys after
    all, the table grows in time: the slots never fill beyond 0.85 and every value matches the oracle."""
    import torch
    announce("no_growth_for_hits", mode)
    rng = np.random.default_rng(77)
    k = 4
    m = {"scalar": capi.MODE_SCALAR, "fixed": capi.MODE_FIXED}[mode]
    om = {"scalar": orc.MODE_SCALAR, "fixed": orc.MODE_FIXED}[mode]
    width = 1 if mode == "scalar" else k
    held = 700000
    # (row storage for every row of the test up front: this is about the slots)
    t = capi.Table(m, initial_capacity=1000000, row_len=k if mode == "fixed" else 0,
                   arena_floats=(held + 700000) * k if mode == "fixed" else 0)
    o = orc.Store(om, k if mode == "fixed" else 0)
    universe = unique_keys(rng, held + 600000)
    base = np.sort(universe[:held])
    fresh = np.sort(universe[held:])
    vals = rng.standard_normal(held * width).astype(np.float32)
    t.push(to_dev(base, dev), to_dev(vals, dev))
    o.push(base, vals)
    t.sync()
    assert t.counters()["slots"] == 1 << 21 and t.counters()["growths"] == 0
    keep = []

    def hits():
        idx = np.sort(rng.choice(held, size=200000, replace=False))
        keys = base[idx]
        v = rng.standard_normal(keys.size * width).astype(np.float32)
        dk, dv = to_dev(keys, dev), to_dev(v, dev)
        keep.append((dk, dv))
        t.push(dk, dv)
        o.push(keys, v)

    # two requests whose records the device has written by the time the next request looks (the GPU is
    # idle, but the table has not been asked to wait): the host has learnt that such requests bring nothing new
    for _ in range(2):
        hits()
        torch.cuda.synchronize()
    for _ in range(80):  # never waited for
        hits()
    c = t.counters()
    assert c["growths"] == 0 and c["waits"] == 0, c
    # now the requests bring new keys after all, 100,000 at a time, still never waited for
    for rep in range(6):
        keys = fresh[rep * 100000:(rep + 1) * 100000]
        v = rng.standard_normal(keys.size * width).astype(np.float32)
        dk, dv = to_dev(keys, dev), to_dev(v, dev)
        keep.append((dk, dv))
        t.push(dk, dv)
        o.push(keys, v)
        assert t.counters()["slots"] * 0.85 >= held + (rep + 1) * 100000  # what the array may hold covers it
    t.sync()
    # the table may have run fuller than its fill limit for those few requests; the next request sees it
    hits()
    t.sync()
    c = t.counters()
    assert c["growths"] >= 1 and c["slots"] * 0.5 >= held + 600000, c
    assert t.size()[0] == o.size()[0] == held + 600000
    gk, gl, gv = t.dump()
    ok, ol, ov = o.dump()
    assert np.array_equal(gk, ok)
    assert_bits_equal(gv, ov, "dump")
    t.close()


@pytest.mark.parametrize("mode", ["scalar", "fixed", "varlen"])
def test_many_requests_in_flight_while_the_table_grows(capi, orc, dev, mode):
    """Device-resident requests are enqueued without waiting, so the host only has bounds on the
    table's counters (every key of a request in flight may be new) and moves them forward from the
    records the device publishes. 240 requests without a single sync from the caller, with key sets
    that repeat, overlap and bring new keys, a table that starts at its minimum size and, for the row
    modes, an arena that starts empty: slots and arena must always have been grown in time."""
    import torch
    announce("requests_in_flight", mode)
    rng = np.random.default_rng({"scalar": 11, "fixed": 12, "varlen": 13}[mode])
    m = {"scalar": capi.MODE_SCALAR, "fixed": capi.MODE_FIXED, "varlen": capi.MODE_VARLEN}[mode]
    om = {"scalar": orc.MODE_SCALAR, "fixed": orc.MODE_FIXED, "varlen": orc.MODE_VARLEN}[mode]
    k = 8
    t = capi.Table(m, initial_capacity=1, row_len=k if mode == "fixed" else 0)
    o = orc.Store(om)
    universe = unique_keys(rng, 60000)
    len_of = rng.choice(np.array([4, 8, 12, 16], np.int32), size=universe.size)
    keep = []  # device buffers of requests in flight must stay alive
    prev = None
    for rep in range(240):
        r = rng.random()
        if prev is not None and r < 0.5:
            idx = prev  # the same keys again: the steady state of a parameter server
        elif r < 0.8:
            lo = int(rng.integers(0, universe.size - 3000))
            idx = np.arange(lo, lo + int(rng.integers(1, 3000)))
        else:
            idx = np.flatnonzero(rng.random(universe.size) < 0.02 * (1 + rep % 5))
        prev = idx
        keys = universe[idx]
        if mode == "scalar":
            lens, vals = None, rng.standard_normal(keys.size).astype(np.float32)
        elif mode == "fixed":
            lens, vals = None, rng.standard_normal(keys.size * k).astype(np.float32)
        else:
            lens = len_of[idx]
            vals = rng.standard_normal(int(lens.sum())).astype(np.float32)
        dk, dv = to_dev(keys, dev), to_dev(vals, dev)
        dl = to_dev(lens, dev) if lens is not None else None
        keep.append((dk, dv, dl))
        t.push(dk, dv, dl)
        o.push(keys, vals, lens)
        if rep % 7 == 3 and mode != "varlen":  # pulls create keys too (not in var-len mode)
            extra = universe[rng.integers(0, universe.size, size=50)]
            extra = np.unique(extra)
            de = to_dev(extra, dev)
            out = torch.empty(extra.size * (k if mode == "fixed" else 1), dtype=torch.float32, device=dev)
            keep.append((de, out, None))
            t.pull(de, out)
            o.pull(extra)
    t.sync()
    _check_dump(t, o, "requests in flight")


def test_tables_driven_from_other_threads(capi, orc, dev):
    """ps-lite calls a request handle on the Customer thread of its KVServer (src/customer.cc:49-63),
    not on the thread that built it, and the servers of different apps run at the same time: four
    tables made here are each driven from a thread of their own, with host buffers, concurrently."""
    import threading
    announce("tables_on_threads")
    modes = [(capi.MODE_SCALAR, orc.MODE_SCALAR), (capi.MODE_FIXED, orc.MODE_FIXED),
             (capi.MODE_VARLEN, orc.MODE_VARLEN), (capi.MODE_SCALAR, orc.MODE_SCALAR)]
    tables = [capi.Table(m, initial_capacity=64, row_len=4 if m == capi.MODE_FIXED else 0) for m, _ in modes]
    failures = []

    def drive(i):
        try:
            t, (m, om) = tables[i], modes[i]
            o = orc.Store(om)
            rng = np.random.default_rng(500 + i)
            universe = unique_keys(rng, 4000)
            lens_all = rng.choice(np.array([4, 8, 20], np.int32), size=universe.size)
            for rep in range(40):
                idx = np.flatnonzero(rng.random(universe.size) < 0.3)
                keys = universe[idx]
                if m == capi.MODE_SCALAR:
                    lens, vals = None, rng.standard_normal(keys.size).astype(np.float32)
                elif m == capi.MODE_FIXED:
                    lens, vals = None, rng.standard_normal(keys.size * 4).astype(np.float32)
                else:
                    lens = lens_all[idx]
                    vals = rng.standard_normal(int(lens.sum())).astype(np.float32)
                t.push(keys, vals, lens)
                o.push(keys, vals, lens)
                if rep % 5 == 4:
                    want, want_lens = o.pull(keys)
                    got = np.zeros(want.size, np.float32)
                    got_lens = np.zeros(keys.size, np.int32) if m == capi.MODE_VARLEN else None
                    t.pull(keys, got, got_lens)
                    assert_bits_equal(got, want, "thread %d pull" % i)
                    if got_lens is not None:
                        assert np.array_equal(got_lens, want_lens)
            # an error on this thread is this thread's: the message names this table's problem
            with pytest.raises(capi.PskvError) as e:
                t.push(universe[:3], np.zeros(7 if m != capi.MODE_VARLEN else 5, np.float32),
                       np.array([1, 2, 3], np.int32) if m == capi.MODE_VARLEN else None)
            assert e.value.code == capi.ESIZE_MISMATCH
            _check_dump(t, o, "thread %d" % i)
        except BaseException as exc:  # noqa: BLE001 - reported on the main thread
            failures.append((i, repr(exc)))

    threads = [threading.Thread(target=drive, args=(i,)) for i in range(len(tables))]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not failures, failures


def test_pinned_pool(capi, orc, dev):
    """pskv_host_alloc / pskv_host_free / pskv_host_trim: buffers are pinned, reusable, may be given
    back from any thread (a ps-lite response is released on a transport thread, zmq_van.h:20-26),
    and serve as request and response buffers of host-resident calls of any size."""
    import threading
    announce("pinned_pool")
    n, k = 40000, 16  # 2.5 MB of values: beyond the size that is served in place
    rng = np.random.default_rng(31)
    keys_np = unique_keys(rng, n)
    pk, pv, po = capi.host_alloc(n * 8), capi.host_alloc(n * k * 4), capi.host_alloc(n * k * 4)
    keys, vals, out = capi.host_array(pk, n, np.uint64), capi.host_array(pv, n * k, np.float32), \
        capi.host_array(po, n * k, np.float32)
    keys[:] = keys_np
    t = capi.Table(capi.MODE_FIXED, initial_capacity=2 * n, row_len=k)
    o = orc.Store(orc.MODE_FIXED, k)
    for rep in range(3):
        vals[:] = rng.standard_normal(n * k).astype(np.float32)
        t.push(keys, vals)
        o.push(keys_np, vals.copy())
    out[:] = 7.0
    assert t.pull(keys, out) == n * k
    assert_bits_equal(out.copy(), o.pull(keys_np)[0], "pull into pinned memory")
    # given back on another thread, the same buffers come out again (same size class)
    th = threading.Thread(target=lambda: [capi.host_free(p) for p in (pv, po)])
    th.start()
    th.join()
    again = {capi.host_alloc(n * k * 4), capi.host_alloc(n * k * 4 - 100)}
    assert again == {pv, po}
    # many threads allocating, writing and freeing at once: no buffer is handed out twice
    seen, lock, errors = [], threading.Lock(), []

    def churn(i):
        try:
            mine = []
            for j in range(50):
                p = capi.host_alloc(4096 * (1 + (i + j) % 5))
                a = capi.host_array(p, 1024, np.uint32)
                a[:] = i * 1000 + j
                mine.append((p, i * 1000 + j))
            for p, tag in mine:
                assert np.all(capi.host_array(p, 1024, np.uint32) == tag), "a buffer was shared"
            with lock:
                seen.extend(p for p, _ in mine)
            for p, _ in mine:
                capi.host_free(p)
        except BaseException as exc:  # noqa: BLE001
            errors.append(repr(exc))

    ths = [threading.Thread(target=churn, args=(i,)) for i in range(8)]
    for th in ths:
        th.start()
    for th in ths:
        th.join()
    assert not errors, errors
    for p in again | {pk}:
        capi.host_free(p)
    capi.host_free(0)          # null is ignored
    capi.host_free(id(seen))   # an address the pool does not know is ignored
    capi.host_trim()
    capi.host_trim()           # nothing left: still fine
    p = capi.host_alloc(1)
    capi.host_array(p, 4096, np.uint8)[:] = 1
    capi.host_free(p)
    capi.host_trim()


@pytest.mark.parametrize("mode", ["scalar", "fixed", "varlen"])
def test_dump_and_size_contract(capi, dev, mode):
    """pskv_size counts keys and floats; pskv_dump with too little room answers PSKV_ESIZE_MISMATCH and
    the sizes it needs, changes nothing, and works without the lens array."""
    import ctypes
    announce("dump_contract", mode)
    m = {"scalar": capi.MODE_SCALAR, "fixed": capi.MODE_FIXED, "varlen": capi.MODE_VARLEN}[mode]
    t = capi.Table(m, initial_capacity=16, row_len=3 if mode == "fixed" else 0)
    assert t.size() == (0, 0)
    assert [a.size for a in t.dump()] == [0, 0, 0]
    keys = np.array([7, 1 << 40, KMAX - 1, KMAX], np.uint64)  # the last one lives in the side slot
    lens = np.array([2, 0, 5, 1], np.int32)
    per = {"scalar": [1, 1, 1, 1], "fixed": [3, 3, 3, 3], "varlen": lens.tolist()}[mode]
    vals = np.arange(1, sum(per) + 1, dtype=np.float32)
    t.push(keys, vals, lens if mode == "varlen" else None)
    assert t.size() == (4, sum(per))
    lib, h = capi.load(), t._h
    nk, nv = ctypes.c_size_t(0), ctypes.c_size_t(0)
    k_small, v_small = np.zeros(3, np.uint64), np.zeros(sum(per), np.float32)
    rc = lib.pskv_dump(h, k_small.ctypes.data, None, 3, v_small.ctypes.data, v_small.size,
                       ctypes.byref(nk), ctypes.byref(nv))
    assert rc == capi.ESIZE_MISMATCH and (nk.value, nv.value) == (4, sum(per))
    k_ok, v_few = np.zeros(4, np.uint64), np.zeros(sum(per) - 1, np.float32)
    rc = lib.pskv_dump(h, k_ok.ctypes.data, None, 4, v_few.ctypes.data, v_few.size,
                       ctypes.byref(nk), ctypes.byref(nv))
    assert rc == capi.ESIZE_MISMATCH and (nk.value, nv.value) == (4, sum(per))
    v_ok = np.zeros(sum(per), np.float32)
    rc = lib.pskv_dump(h, k_ok.ctypes.data, None, 4, v_ok.ctypes.data, v_ok.size, ctypes.byref(nk), ctypes.byref(nv))
    assert rc == capi.OK and (nk.value, nv.value) == (4, sum(per))
    assert k_ok.tolist() == keys.tolist()  # sorted by key, the side slot's key last
    assert np.array_equal(v_ok, vals)      # 0.0f + v for every float, rows in key order
    gk, gl, gv = t.dump()
    assert gk.tolist() == keys.tolist() and gl.tolist() == per and np.array_equal(gv, vals)
    assert t.size() == (4, sum(per))


def test_misuse_is_a_status_code(capi, dev):
    """The C ABI never throws and never crashes on misuse: bad creation arguments, null handles and null
    buffers come back as PSKV_EINVAL with a message."""
    import ctypes
    announce("misuse")
    for kw in ({"mode": 7}, {"mode": -1}, {"max_load": 0.95}, {"max_load": -0.1}, {"device": 99}, {"device": -1}):
        with pytest.raises(capi.PskvError) as e:
            capi.Table(**kw)
        assert e.value.code == capi.EINVAL, kw
    lib = capi.load()
    h = ctypes.c_void_p()
    assert lib.pskv_table_create(ctypes.byref(h), None) == capi.EINVAL
    assert lib.pskv_table_create(None, None) == capi.EINVAL
    assert lib.pskv_table_destroy(None) == capi.OK
    null = ctypes.c_void_p()
    n1 = ctypes.c_size_t(0)
    assert lib.pskv_push(null, None, 0, None, 0, None, 0, capi.MEM_HOST) == capi.EINVAL
    assert lib.pskv_pull(null, None, 0, None, 0, None, ctypes.byref(n1), capi.MEM_HOST) == capi.EINVAL
    assert lib.pskv_sync(null) == capi.EINVAL
    assert b"null" in lib.pskv_last_error()
    t = capi.Table(capi.MODE_SCALAR)
    keys = np.array([1, 2, 3], np.uint64)
    assert lib.pskv_push(t._h, None, 3, None, 3, None, 0, capi.MEM_HOST) == capi.EINVAL       # null keys
    assert lib.pskv_push(t._h, keys.ctypes.data, 3, None, 3, None, 0, capi.MEM_HOST) == capi.EINVAL  # null vals
    assert lib.pskv_push(t._h, keys.ctypes.data, 3, None, 3, None, 0, 5) == capi.EINVAL       # bad memkind
    assert lib.pskv_pull(t._h, keys.ctypes.data, 3, None, 3, None, None, capi.MEM_HOST) == capi.EINVAL  # null out
    assert lib.pskv_push(t._h, None, 0, None, 0, None, 0, capi.MEM_HOST) == capi.OK           # an empty request is fine
    assert lib.pskv_pull(t._h, None, 0, None, 0, None, ctypes.byref(n1), capi.MEM_HOST) == capi.OK and n1.value == 0
    assert lib.pskv_last_error() == b""  # a successful call clears the message
    assert t.size() == (0, 0)


def test_device_time_accounting(capi, dev):
    """pskv_prof_*: every launch of the listed kernels is timed by its own pair of events; the samples
    add up to the total, and the copy probe moves what it says."""
    import torch
    announce("prof")
    n = 100000
    keys = to_dev(unique_keys(np.random.default_rng(3), n), dev)
    vals = torch.ones(n, dtype=torch.float32, device=dev)
    out = torch.zeros(n, dtype=torch.float32, device=dev)
    t = capi.Table(capi.MODE_SCALAR, initial_capacity=2 * n)
    t.push(keys, vals)  # not counted: profiling is off
    t.prof_enable(True)
    t.prof_reset()
    for _ in range(5):
        t.push(keys, vals)
    t.pull(keys, out)
    src = torch.arange(1 << 20, dtype=torch.float32, device=dev)
    dst = torch.zeros(1 << 20, dtype=torch.float32, device=dev)
    t.copy_probe(dst, src)
    launches, total_ms = t.prof_read(capi.KERNEL_PUSH_SCALAR)
    samples = t.prof_samples(capi.KERNEL_PUSH_SCALAR)
    assert launches == 5 and samples.size == 5
    assert np.all(samples > 0) and abs(float(samples.sum()) - total_ms) < 1e-3 * max(total_ms, 1e-3) + 1e-4
    assert t.prof_read(capi.KERNEL_PULL_SCALAR)[0] == 1
    assert t.prof_read(capi.KERNEL_COPY)[0] == 1
    assert torch.equal(dst, src)
    assert np.all(from_dev(out) == 6.0)
    t.prof_enable(False)
    t.push(keys, vals)
    assert t.prof_read(capi.KERNEL_PUSH_SCALAR)[0] == 5
    t.prof_reset()
    assert t.prof_read(capi.KERNEL_PUSH_SCALAR) == (0, 0.0) and t.prof_samples(capi.KERNEL_PUSH_SCALAR).size == 0


def test_scalar_size_checks(capi, dev):
    announce("scalar_size_checks")
    t = capi.Table(capi.MODE_SCALAR)
    keys = np.array([1, 2, 3], np.uint64)
    with pytest.raises(capi.PskvError) as e:  # kv_app.h:447
        t.push(keys, np.zeros(2, np.float32))
    assert e.value.code == capi.ESIZE_MISMATCH
    out = np.zeros(2, np.float32)
    with pytest.raises(capi.PskvError) as e:
        t.pull(keys, out)
    assert e.value.code == capi.ESIZE_MISMATCH and t.last_out_nvals == 3
    assert t.size() == (3, 3)  # the pull still created the keys, as the reference would
    t.push(np.zeros(0, np.uint64), np.zeros(0, np.float32))
    assert t.pull(np.zeros(0, np.uint64), np.zeros(0, np.float32)) == 0


@pytest.mark.parametrize("memkind", ["device", "host"])
@pytest.mark.parametrize("n,k", [(64, 4096 * 3), (5, 1), (1000, 2), (300, 7), (257, 64), (3, 100000),
                                 (2, 4096 + 8)])
def test_fixed_rows(capi, orc, dev, memkind, n, k):
    import torch
    announce("fixed_rows", memkind, n, k)
    rng = np.random.default_rng(n * 131 + k)
    t = capi.Table(capi.MODE_FIXED, initial_capacity=16)
    o = orc.Store(orc.MODE_FIXED)
    universe = unique_keys(rng, 2 * n)
    for rep in range(3):
        keys = np.sort(rng.choice(universe, size=n, replace=False))
        vals = rng.uniform(-1, 1, size=n * k).astype(np.float32)
        if rep == 0:
            vals[: min(8, vals.size)] = -0.0
        if memkind == "device":
            t.push(to_dev(keys, dev), to_dev(vals, dev))
        else:
            t.push(keys, vals)
        o.push(keys, vals)
    keys = np.sort(rng.choice(universe, size=n, replace=False))
    want, _ = o.pull(keys)
    if memkind == "device":
        out = torch.full((n * k,), 7.0, dtype=torch.float32, device=dev)
        assert t.pull(to_dev(keys, dev), out) == n * k
        t.sync()
        got = from_dev(out)
    else:
        got = np.full(n * k, 7.0, np.float32)
        assert t.pull(keys, got) == n * k
    assert_bits_equal(got, want, "fixed pull")
    # push+pull in one request
    vals = rng.uniform(-1, 1, size=n * k).astype(np.float32)
    want, _ = o.pushpull(keys, vals)
    got = np.zeros(n * k, np.float32)
    t.pushpull(keys, vals, got)
    assert_bits_equal(got, want, "fixed pushpull")
    _check_dump(t, o, "fixed")


def test_fixed_errors(capi, dev):
    announce("fixed_errors")
    t = capi.Table(capi.MODE_FIXED)
    keys = np.array([1, 2, 3], np.uint64)
    with pytest.raises(capi.PskvError) as e:  # row length still unknown
        t.pull(keys, np.zeros(3, np.float32))
    assert e.value.code == capi.EINVAL
    with pytest.raises(capi.PskvError) as e:  # kv_app.h:549
        t.push(keys, np.zeros(7, np.float32))
    assert e.value.code == capi.ESIZE_MISMATCH
    t.push(keys, np.ones(6, np.float32))
    with pytest.raises(capi.PskvError) as e:
        t.push(keys, np.ones(9, np.float32))
    assert e.value.code == capi.ESIZE_MISMATCH
    got = np.zeros(6, np.float32)
    t.pull(keys, got)
    assert np.array_equal(got, np.ones(6, np.float32))


LENS_SETS = {
    "emb": [8, 16, 32, 64, 128],
    "ragged": [0, 1, 2, 3, 5, 7, 9, 31],
    "mult4": [0, 4, 4, 4, 8],
    "long": [4, 20000, 8, 4096, 12],
}


@pytest.mark.parametrize("memkind", ["device", "host"])
@pytest.mark.parametrize("n,lens_set", [(2000, "emb"), (5000, "ragged"), (9000, "mult4"),
                                        (40, "long"), (1, "emb")])
def test_varlen_rows(capi, orc, dev, memkind, n, lens_set):
    import torch
    announce("varlen_rows", memkind, n, lens_set)
    rng = np.random.default_rng(n + len(lens_set))
    t = capi.Table(capi.MODE_VARLEN, initial_capacity=16)
    o = orc.Store(orc.MODE_VARLEN)
    universe = unique_keys(rng, 2 * n)
    len_of = dict(zip(universe.tolist(),
                      rng.choice(np.array(LENS_SETS[lens_set], np.int32), size=universe.size).tolist()))
    for rep in range(3):
        keys = np.sort(rng.choice(universe, size=n, replace=False))
        lens = np.array([len_of[k] for k in keys.tolist()], np.int32)
        vals = rng.normal(0, 0.1, size=int(lens.sum())).astype(np.float32)
        if memkind == "device":
            t.push(to_dev(keys, dev), to_dev(vals, dev), to_dev(lens, dev))
        else:
            t.push(keys, vals, lens)
        o.push(keys, vals, lens)
    keys = np.sort(rng.choice(universe, size=n, replace=False))  # some absent: len 0, not created
    want, want_lens = o.pull(keys)
    if memkind == "device":
        out = torch.full((want.size + 5,), 7.0, dtype=torch.float32, device=dev)
        out_lens = torch.full((n,), -1, dtype=torch.int32, device=dev)
        got_n = t.pull(to_dev(keys, dev), out, out_lens)
        t.sync()
        got, got_lens = from_dev(out)[:got_n], from_dev(out_lens)
    else:
        got = np.full(want.size, 7.0, np.float32)
        got_lens = np.full(n, -1, np.int32)
        got_n = t.pull(keys, got, got_lens)
    assert got_n == want.size
    assert np.array_equal(got_lens, want_lens)
    assert_bits_equal(got, want, "varlen pull")
    _check_dump(t, o, "varlen")


def test_varlen_errors(capi, orc, dev):
    announce("varlen_errors")
    t = capi.Table(capi.MODE_VARLEN)
    o = orc.Store(orc.MODE_VARLEN)
    keys = np.array([10, 20, 30], np.uint64)
    lens = np.array([2, 0, 3], np.int32)
    vals = np.arange(5, dtype=np.float32)
    for s in (t, o):
        s.push(keys, vals, lens)
    # host-visible checks
    with pytest.raises(capi.PskvError) as e:
        t.push(keys, vals, lens[:2])
    assert e.value.code == capi.ESIZE_MISMATCH
    with pytest.raises(capi.PskvError) as e:
        t.push(keys, vals[:4], lens)
    assert e.value.code == capi.ESIZE_MISMATCH
    with pytest.raises(capi.PskvError) as e:
        t.push(keys, vals, np.array([2, -1, 4], np.int32))
    assert e.value.code == capi.EINVAL
    # a changed length is refused: nothing stored changes, absent keys become zero rows
    keys2 = np.array([10, 25, 30], np.uint64)
    lens2 = np.array([2, 4, 1], np.int32)
    vals2 = np.ones(7, np.float32)
    with pytest.raises(capi.PskvError) as e:
        t.push(keys2, vals2, lens2)
    assert e.value.code == capi.ELEN_CHANGED
    assert o.handle(True, False, keys2, vals2, lens2)[0] == orc.ELEN_CHANGED
    _check_dump(t, o, "after refused push")
    # the same through device buffers: the error is reported by the next sync
    keys3 = np.array([10, 26, 30], np.uint64)
    t.push(to_dev(keys3, dev), to_dev(vals2, dev), to_dev(lens2, dev))
    with pytest.raises(capi.PskvError) as e:
        t.sync()
    assert e.value.code == capi.ELEN_CHANGED
    assert o.handle(True, False, keys3, vals2, lens2)[0] == orc.ELEN_CHANGED
    t.sync()  # reported once
    _check_dump(t, o, "after refused device push")
    # response too small
    out = np.zeros(2, np.float32)
    with pytest.raises(capi.PskvError) as e:
        t.pull(keys, out, np.zeros(3, np.int32))
    assert e.value.code == capi.ESIZE_MISMATCH and t.last_out_nvals == 5


def test_refused_push_still_publishes_its_counters(capi, orc, dev):
    """Close to a limit the host asks the request's own kernel for the counters as they are after
    it, and sizes the next request from that record instead of waiting for the stream. A var-len
    push that the device refuses (its lens do not add up to the values it brought) changes no
    counter but must leave its record all the same, or the host would count its keys as pending
    for good and wait for exact counters before every later request."""
    import time
    announce("refused_push_publishes")
    rng = np.random.default_rng(321)
    n, row = 1000, 16
    keys = [unique_keys(rng, n) for _ in range(3)]
    lens = np.full(n, row, np.int32)
    vals = rng.integers(-5, 5, size=n * row).astype(np.float32)
    # room for two requests and a half by the host's upper bound (rows + one unit per key + padding)
    t = capi.Table(capi.MODE_VARLEN, initial_capacity=8 * n, arena_floats=52000)
    o = orc.Store(orc.MODE_VARLEN)
    t.push(to_dev(keys[0], dev), to_dev(vals, dev), to_dev(lens, dev))
    o.push(keys[0], vals, lens)
    t.sync()
    before = t.counters()
    t.push(to_dev(keys[1], dev), to_dev(vals[:-4], dev), to_dev(lens, dev))  # four floats short: refused on the device
    time.sleep(0.05)  # (the device gets there; nothing here waits for it)
    t.push(to_dev(keys[2], dev), to_dev(vals, dev), to_dev(lens, dev))
    o.push(keys[2], vals, lens)
    after = t.counters()
    assert after["waits"] == before["waits"], (before, after)
    assert after["growths"] == before["growths"], (before, after)
    with pytest.raises(capi.PskvError) as e:
        t.sync()
    assert e.value.code == capi.ESIZE_MISMATCH
    t.sync()
    _check_dump(t, o, "after the refused push")


def test_varlen_pull_without_host_round_trip(capi, orc, dev):
    """out_nvals == NULL keeps a var-len pull asynchronous: the kernels take the response size from
    the device-side scan. Too small a buffer writes nothing and is reported by the next sync."""
    import torch
    announce("varlen_async_pull")
    rng = np.random.default_rng(44)
    n = 30000
    keys = unique_keys(rng, n)
    lens = rng.choice(np.array([0, 8, 16, 24, 200], np.int32), size=n).astype(np.int32)
    vals = rng.normal(0, 1, size=int(lens.sum())).astype(np.float32)
    t = capi.Table(capi.MODE_VARLEN, initial_capacity=1024)
    o = orc.Store(orc.MODE_VARLEN)
    dk, dl = to_dev(keys, dev), to_dev(lens, dev)
    for _ in range(2):
        t.push(dk, to_dev(vals, dev), dl)
        o.push(keys, vals, lens)
    probe = np.sort(np.concatenate([keys[::2], unique_keys(rng, 500)]))
    probe = np.unique(probe)
    want, want_lens = o.pull(probe)
    dp = to_dev(probe, dev)
    out = torch.full((want.size + 4096,), 7.0, dtype=torch.float32, device=dev)  # more room than needed
    out_lens = torch.full((probe.size,), -1, dtype=torch.int32, device=dev)
    torch.cuda.synchronize()  # raw pointers: torch's fills above must have landed
    t.pull_raw(dp.data_ptr(), probe.size, out.data_ptr(), out.numel(), out_lens.data_ptr())
    t.sync()
    assert np.array_equal(from_dev(out_lens), want_lens)
    assert_bits_equal(from_dev(out)[:want.size], want, "async pull")
    assert np.all(from_dev(out)[want.size:] == 7.0)  # nothing written past the response
    small = torch.full((want.size - 8,), 7.0, dtype=torch.float32, device=dev)
    torch.cuda.synchronize()
    t.pull_raw(dp.data_ptr(), probe.size, small.data_ptr(), small.numel(), out_lens.data_ptr())
    with pytest.raises(capi.PskvError) as e:
        t.sync()
    assert e.value.code == capi.ESIZE_MISMATCH
    assert np.all(from_dev(small) == 7.0)
    t.sync()
    _check_dump(t, o, "after async pulls")


@pytest.mark.parametrize("memkind", ["device", "host"])
@pytest.mark.parametrize("nkeys,row", [(40, 24), (3000, 8), (9000, 72)])
def test_varlen_tiles_in_two_arena_pieces(capi, orc, dev, memkind, nkeys, row):
    """A request that repeats the cached one maps a 256-float tile through the note its predecessor
    left: one arena piece, or two. Here the upper half of the keys is created first and the lower
    half second, so in a request over all keys the tile around the middle lies in two pieces and
    the second piece sits BELOW the first in the arena (a negative distance); further pieces come
    from the lookup's workgroups. Pushes and pulls that repeat that request must give the
    oracle's sums; then a changed length in the middle must end the shortcut."""
    import torch
    announce("varlen_two_pieces", memkind, nkeys, row)
    rng = np.random.default_rng(nkeys + row)
    keys = unique_keys(rng, nkeys)
    lens = np.full(nkeys, row, np.int32)
    lens[rng.integers(0, nkeys, size=nkeys // 10)] = 0      # rows without floats in between
    lens[rng.integers(0, nkeys, size=nkeys // 10)] = 4 * row
    half = nkeys // 2
    t = capi.Table(capi.MODE_VARLEN, initial_capacity=64)
    o = orc.Store(orc.MODE_VARLEN)

    def push(k, l):
        v = rng.integers(-8, 8, size=int(l.sum())).astype(np.float32)
        if memkind == "device":
            t.push(to_dev(k, dev), to_dev(v, dev), to_dev(l, dev))
        else:
            t.push(k, v, l)
        o.push(k, v, l)

    def pull_and_check(k, what):
        want, want_lens = o.pull(k)
        got = np.full(want.size, 7.0, np.float32)
        got_lens = np.full(k.size, -1, np.int32)
        if memkind == "device":
            out = torch.full((want.size,), 7.0, dtype=torch.float32, device=dev)
            out_lens = torch.full((k.size,), -1, dtype=torch.int32, device=dev)
            t.pull(to_dev(k, dev), out, out_lens)
            t.sync()
            got, got_lens = from_dev(out), from_dev(out_lens)
        else:
            t.pull(k, got, got_lens)
        assert np.array_equal(got_lens, want_lens), what
        assert_bits_equal(got, want, what)

    push(keys[half:], lens[half:])
    push(keys[:half], lens[:half])
    for rep in range(4):          # the first writes the notes, the others use them
        push(keys, lens)
        pull_and_check(keys, "repeat %d" % rep)
    pull_and_check(keys, "pull again")
    sub = keys[half - 5:half + 5]
    push(sub, lens[half - 5:half + 5])
    for rep in range(2):
        push(keys, lens)
        pull_and_check(keys, "after another request %d" % rep)
    _check_dump(t, o, "two pieces")


@pytest.mark.parametrize("mode", ["scalar", "fixed", "varlen"])
def test_duplicate_keys_do_no_harm(capi, dev, mode):
    """Keys of a request must be unique (kv_app.h:17). A request that repeats a key is a caller error:
    the row modes report it, and in no mode does it touch memory it should not."""
    announce("duplicate_keys", mode)
    keys = np.array([5, 9, 9, 9, 12, 12, 40], np.uint64)
    m = {"scalar": capi.MODE_SCALAR, "fixed": capi.MODE_FIXED, "varlen": capi.MODE_VARLEN}[mode]
    t = capi.Table(m, initial_capacity=16)
    if mode == "scalar":
        # sorted repeats even have the reference's result, see test_scalar_sorted_repeats
        t.push(keys, np.ones(keys.size, np.float32))
        out = np.zeros(keys.size, np.float32)
        t.pull(keys, out)
        assert t.size()[0] == 4
        assert np.array_equal(out, [1, 3, 3, 3, 2, 2, 1])
        # unsorted repeats: which of the racing adds survives is unspecified, memory stays sound
        mixed = np.array([9, 5, 9, 40, 5, 9, 77], np.uint64)
        t.push(mixed, np.ones(mixed.size, np.float32))
        assert t.size()[0] == 5
        return
    lens = np.full(keys.size, 8, np.int32)
    try:
        t.push(keys, np.ones(keys.size * 8, np.float32), lens if mode == "varlen" else None)
        reported = False
    except capi.PskvError as e:
        reported = e.code == capi.EINVAL
    assert reported
    # the refused request changed no value; FIXED has created the keys it named as zero rows (as a
    # pull of them would), VARLEN has created nothing
    assert t.size()[0] == (4 if mode == "fixed" else 0)
    # the table is still usable
    uniq = np.unique(keys)
    t.push(uniq, np.ones(uniq.size * 8, np.float32), np.full(uniq.size, 8, np.int32) if mode == "varlen" else None)
    out = np.zeros(uniq.size * 8, np.float32)
    t.pull(uniq, out, np.zeros(uniq.size, np.int32) if mode == "varlen" else None)
    assert np.all(out >= 1.0)


@pytest.mark.parametrize("memkind", ["device", "host"])
@pytest.mark.parametrize("n", [7, 300, 100000])
def test_scalar_sorted_repeats(capi, orc, dev, memkind, n):
    """The reference's handle is a plain loop over the request (kv_app.h:451-459): a sorted request
    that repeats a key adds the values in request order and every pulled position shows the sum so
    far. Runs of every length, runs that cross wavefront and workgroup boundaries, a run at the very
    start and one at the very end, through push, pull and push+pull."""
    import torch
    announce("scalar_sorted_repeats", memkind, n)
    rng = np.random.default_rng(n)
    t = capi.Table(capi.MODE_SCALAR, initial_capacity=16)
    o = orc.Store(orc.MODE_SCALAR)
    universe = unique_keys(rng, n)
    for rep in range(5):
        reps = rng.choice([1, 1, 1, 2, 3, 70, 300], size=n)
        keys = np.sort(np.repeat(universe, reps)[:n] if rep % 2 == 0 else
                       np.repeat(universe[::-1], reps)[-n:])
        if rep == 4:
            keys = np.full(n, universe[0], np.uint64)  # one run over the whole request
        vals = rng.standard_normal(n).astype(np.float32)
        want = o.handle(True, True, keys, vals, out_cap=n)[1]
        if memkind == "device":
            out = torch.full((n,), 7.0, dtype=torch.float32, device=dev)
            t.pushpull(to_dev(keys, dev), to_dev(vals, dev), out)
            t.sync()
            got = from_dev(out)
        else:
            got = np.full(n, 7.0, np.float32)
            t.pushpull(keys, vals, got)
        assert_bits_equal(got, want, "push+pull %d" % rep)
        vals = rng.standard_normal(n).astype(np.float32)
        t.push(to_dev(keys, dev), to_dev(vals, dev)) if memkind == "device" else t.push(keys, vals)
        o.push(keys, vals)
        got = np.full(n, 7.0, np.float32)
        t.pull(keys, got)
        assert_bits_equal(got, o.pull(keys)[0], "pull %d" % rep)
    _check_dump(t, o, "sorted repeats")


@pytest.fixture
def small_scalar_cache(monkeypatch):
    """Tables created in the test let SCALAR requests of 64 keys and more use the key cache (the
    default is 131,072), so that short sequences of small requests go through all of its states."""
    monkeypatch.setenv("PSKV_SCALAR_CACHE_MIN_KEYS", "64")


def _drive_key_sets(capi, orc, dev, mode, seed, steps, script="random"):
    """One random sequence of requests over a few related key sets, through every entry point and
    both memory kinds, every pull compared with the oracle, the dump at the end. `script` shapes
    the sequence: "random" draws the key set of every step from all of them; "two_sizes" alternates
    between two sets of different sizes (each recorded in turn); "threshold" mixes sets below and
    above the size from which SCALAR requests use the key cache; "growth" keeps bringing sets of
    new keys between repeats of one set, so that the table grows while that set is cached."""
    import torch
    rng = np.random.default_rng(1000 + seed)
    n = int(rng.integers(300, 3000)) if script != "threshold" else int(rng.integers(80, 200))
    k = 1 if mode == "scalar" else 8
    base = unique_keys(rng, n + 50)
    sets = {}
    sets["A"] = base[:n].copy()
    b = base[:n].copy()
    b[int(rng.integers(0, n))] = base[n + 1]  # one key differs
    sets["B"] = np.sort(b)
    sets["C"] = base[10:n + 10].copy()        # same size, shifted
    sets["D"] = base[: n // 2].copy()         # a different size
    names = ["A", "A", "A", "B", "C", "D", "A"]
    extra_keys = np.zeros(0, np.uint64)
    if mode == "scalar" and script == "random":
        sets["E"] = np.union1d(base, unique_keys(rng, 6 * n))  # makes the table grow when it first comes
        names += ["E"]
    if script == "two_sizes":
        names = ["A", "D"]
    if script == "threshold":  # (the fixture sets the threshold to 64 keys)
        sets["F"] = base[:40].copy()
        sets["G"] = base[5:68].copy()   # one key below the threshold
        sets["H"] = base[5:69].copy()   # exactly at it
        names = ["A", "F", "G", "H", "A", "H", "F"]
    if script == "growth":
        extra_keys = unique_keys(rng, 40 * n)
        names = ["A", "A", "new", "A", "new", "B"]
    pool = np.union1d(base, extra_keys)
    lens_of = {int(key): int(l) for key, l in zip(pool.tolist(), rng.choice([0, 4, 8, 12, 40], size=pool.size))}
    m = {"scalar": capi.MODE_SCALAR, "fixed": capi.MODE_FIXED, "varlen": capi.MODE_VARLEN}[mode]
    om = {"scalar": orc.MODE_SCALAR, "fixed": orc.MODE_FIXED, "varlen": orc.MODE_VARLEN}[mode]
    t = capi.Table(m, initial_capacity=64, row_len=k if mode == "fixed" else 0)  # small: the slot array grows during the sequence
    o = orc.Store(om, k if mode == "fixed" else 0)

    def lens_for(keys):
        return np.array([lens_of[int(x)] for x in keys.tolist()], np.int32) if mode == "varlen" else None

    fresh_at = 0
    for step in range(steps):
        name = names[step % 2] if script == "two_sizes" and step < steps // 2 else names[int(rng.integers(0, len(names)))]
        if name == "new":
            keys = extra_keys[fresh_at:fresh_at + n]
            fresh_at = (fresh_at + n) % (extra_keys.size - n)
        else:
            keys = sets[name]
        lens = lens_for(keys)
        nvals = int(lens.sum()) if mode == "varlen" else keys.size * k
        op = ["push", "push", "pull", "pull_async", "pushpull"][int(rng.integers(0, 5))]
        on_dev = bool(rng.integers(0, 2))
        vals = rng.integers(-8, 8, size=nvals).astype(np.float32)
        if mode == "scalar":
            vals = rng.normal(0, 1, size=nvals).astype(np.float32)  # sums that depend on their order
        kk = to_dev(keys, dev) if on_dev else keys
        vv = to_dev(vals, dev) if on_dev else vals
        ll = None if lens is None else (to_dev(lens, dev) if on_dev else lens)
        what = "seed %d %s step %d %s %s %s" % (seed, script, step, op, name, "dev" if on_dev else "host")
        if op == "push":
            t.push(kk, vv, ll)
            o.push(keys, vals, lens)
        elif op == "pushpull":
            want, want_lens = o.pushpull(keys, vals, lens)
            if on_dev:
                out = torch.full((nvals,), 7.0, dtype=torch.float32, device=dev)
                out_lens = torch.full((keys.size,), -1, dtype=torch.int32, device=dev)
                t.pushpull(kk, vv, out, ll, out_lens if mode == "varlen" else None)
                t.sync()
                got, got_lens = from_dev(out), from_dev(out_lens)
            else:
                got = np.full(nvals, 7.0, np.float32)
                got_lens = np.full(keys.size, -1, np.int32)
                t.pushpull(keys, vals, got, lens, got_lens if mode == "varlen" else None)
            assert_bits_equal(got, want, what)
            if mode == "varlen":
                assert np.array_equal(got_lens, want_lens), what
        else:
            want, want_lens = o.pull(keys)
            if op == "pull_async":
                dk = to_dev(keys, dev)
                out = torch.full((want.size + 64,), 7.0, dtype=torch.float32, device=dev)
                out_lens = torch.full((keys.size,), -1, dtype=torch.int32, device=dev)
                torch.cuda.synchronize()  # raw pointers: torch's fills above must have landed
                t.pull_raw(dk.data_ptr(), keys.size, out.data_ptr(), out.numel(),
                           out_lens.data_ptr() if mode == "varlen" else None)
                t.sync()
                got, got_lens = from_dev(out)[:want.size], from_dev(out_lens)
            elif on_dev:
                out = torch.full((want.size,), 7.0, dtype=torch.float32, device=dev)
                out_lens = torch.full((keys.size,), -1, dtype=torch.int32, device=dev)
                assert t.pull(kk, out, out_lens if mode == "varlen" else None) == want.size
                t.sync()
                got, got_lens = from_dev(out), from_dev(out_lens)
            else:
                got = np.full(want.size, 7.0, np.float32)
                got_lens = np.full(keys.size, -1, np.int32)
                assert t.pull(keys, got, got_lens if mode == "varlen" else None) == want.size
            assert_bits_equal(got, want, what)
            if mode == "varlen":
                assert np.array_equal(got_lens, want_lens), what
    t.sync()
    _check_dump(t, o, "seed %d %s after the sequence" % (seed, script))
    t.close()


@pytest.mark.parametrize("mode", ["scalar", "fixed", "varlen"])
@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_repeated_and_alternating_key_sets(capi, orc, dev, mode, seed, small_scalar_cache):
    """Requests that repeat the previous request's keys take a path that skips the hash probes; requests
    that do not must never see what that path left behind. Random sequences over a few key sets that
    are equal, differ in one key, differ in one length or differ in size, through every entry point
    and both memory kinds, checked against the oracle after every pull. (SCALAR: the values of a
    repeated key set live in a request-ordered array that is ahead of the slots until something else
    needs them; a larger key set makes the table grow in the middle of that.)"""
    announce("repeated_key_sets", mode, seed)
    _drive_key_sets(capi, orc, dev, mode, seed, 60 if mode == "scalar" else 40)


@pytest.mark.parametrize("mode", ["scalar", "fixed", "varlen"])
def test_key_cache_policy_over_many_sequences(capi, orc, dev, mode, small_scalar_cache):
    """What decides whether a request is compared with, served from or recorded into the key cache
    is host-side bookkeeping (sizes that repeat, pulls that follow pushes, comparisons that keep
    failing, the size threshold). 256 further sequences per mode, a quarter each of four shapes: any
    key set at any step; two sets of different sizes in strict alternation, then at random; sets
    just below, at and above the threshold; new keys that make the table grow between repeats of
    a cached set. Stops at the first sequence that differs from the oracle."""
    import time
    announce("key_cache_policy", mode)
    scripts = ["random", "two_sizes", "threshold", "growth"]
    t0 = time.time()
    for seed in range(100, 356):
        _drive_key_sets(capi, orc, dev, mode, seed, 40, scripts[seed % 4])
    print("256 sequences in %.1f s" % (time.time() - t0), flush=True)


def test_refused_push_does_not_poison_repeats(capi, orc, dev):
    """A var-len push refused for a changed length must not leave anything behind that a repeat of the
    same keys could pick up."""
    announce("refused_push_then_repeat")
    rng = np.random.default_rng(9)
    keys = unique_keys(rng, 500)
    lens = rng.choice(np.array([4, 8, 16], np.int32), size=500).astype(np.int32)
    bad = lens.copy()
    bad[123] += 4
    t = capi.Table(capi.MODE_VARLEN, initial_capacity=64)
    o = orc.Store(orc.MODE_VARLEN)
    dk, dl, dbad = to_dev(keys, dev), to_dev(lens, dev), to_dev(bad, dev)
    for which in ("good", "good", "bad", "bad", "good", "good"):
        l, dlx = (lens, dl) if which == "good" else (bad, dbad)
        vals = rng.integers(-4, 4, size=int(l.sum())).astype(np.float32)
        t.push(dk, to_dev(vals, dev), dlx)
        rc = o.handle(True, False, keys, vals, l)[0]
        if which == "bad":
            assert rc == orc.ELEN_CHANGED
            with pytest.raises(capi.PskvError) as e:
                t.sync()
            assert e.value.code == capi.ELEN_CHANGED
        else:
            assert rc == 0
            t.sync()
        out = np.zeros(int(lens.sum()), np.float32)
        out_lens = np.zeros(500, np.int32)
        t.pull(keys, out, out_lens)
        want, want_lens = o.pull(keys)
        assert np.array_equal(out_lens, want_lens)
        assert_bits_equal(out, want, "after a %s push" % which)


def test_scalar_long_probe_chains(capi, orc, dev):
    """A nearly full slot array (fill 0.9) makes colliding keys walk long probe sequences; results and
    the stored key set stay exact, and growth still happens before the array is full."""
    announce("scalar_long_probes")
    rng = np.random.default_rng(31)
    t = capi.Table(capi.MODE_SCALAR, initial_capacity=900, max_load=0.9)
    o = orc.Store(orc.MODE_SCALAR)
    universe = unique_keys(rng, 20000)
    for rep in range(30):
        keys = np.sort(rng.choice(universe, size=int(rng.integers(1, 900)), replace=False))
        vals = rng.integers(-100, 100, size=keys.size).astype(np.float32)
        t.push(to_dev(keys, dev), to_dev(vals, dev))
        o.push(keys, vals)
        if rep % 5 == 4:
            probe = np.sort(rng.choice(universe, size=700, replace=False))
            got = np.zeros(700, np.float32)
            t.pull(probe, got)
            assert_bits_equal(got, o.pull(probe)[0], "rep %d" % rep)
    _check_dump(t, o, "long probes")


def _row_push(t, dev, memkind, keys, vals, lens):
    """A push through host or device buffers; returns the status the caller gets to see (device
    buffers: at the next sync)."""
    try:
        if memkind == "device":
            t.push(to_dev(keys, dev), to_dev(vals, dev), None if lens is None else to_dev(lens, dev))
            t.sync()
        else:
            t.push(keys, vals, lens)
    except Exception as e:  # capi.PskvError
        return e.code
    return 0


@pytest.mark.parametrize("memkind", ["device", "host"])
@pytest.mark.parametrize("mode", ["fixed", "varlen"])
def test_sorted_repeats_refuse_row_requests(capi, orc, dev, mode, memkind):
    """Keys of a request are sorted and unique (kv_app.h:17). In the row modes a sorted request that
    repeats a key is refused as a whole with PSKV_EINVAL, whether the key is new or already stored and
    wherever in the request the repeat sits: no stored value changes. (A FIXED request may leave
    keys it named as zero rows, as a pull of them would.)"""
    announce("sorted_repeats_refused", mode, memkind)
    rng = np.random.default_rng(91)
    m = capi.MODE_FIXED if mode == "fixed" else capi.MODE_VARLEN
    om = orc.MODE_FIXED if mode == "fixed" else orc.MODE_VARLEN
    k = 8
    t = capi.Table(m, initial_capacity=16)
    o = orc.Store(om)

    def lens_for(n):
        return None if mode == "fixed" else np.full(n, k, np.int32)

    base = unique_keys(rng, 700)
    vals = rng.normal(0, 1, size=base.size * k).astype(np.float32)
    assert _row_push(t, dev, memkind, base, vals, lens_for(base.size)) == 0
    o.push(base, vals, lens_for(base.size))
    _check_dump(t, o, "before")

    def refused(keys):
        v = np.ones(keys.size * k, np.float32)
        assert _row_push(t, dev, memkind, keys, v, lens_for(keys.size)) == capi.EINVAL
        if mode == "fixed":
            o.pull(np.unique(keys))  # a FIXED pull creates absent keys as zero rows
        _check_dump(t, o, "after a refused request")

    # the very key the table already holds, twice
    refused(np.array([base[9], base[9]], np.uint64))
    # a repeat of a stored key one workgroup apart (positions 255 and 256), among stored keys
    refused(np.concatenate([base[:256], base[255:600]]))
    # a repeat of a NEW key, at the wavefront boundary 63/64 and at the end of the request
    fresh = unique_keys(rng, 300)
    fresh = np.setdiff1d(fresh, base)[:200]
    refused(np.concatenate([fresh[:64], fresh[63:150], fresh[149:150]]))
    # a long run
    refused(np.sort(np.concatenate([base[:5], np.full(300, base[3], np.uint64)])))
    # the table still serves good requests, and they see the values of before
    more = rng.normal(0, 1, size=base.size * k).astype(np.float32)
    assert _row_push(t, dev, memkind, base, more, lens_for(base.size)) == 0
    o.push(base, more, lens_for(base.size))
    _check_dump(t, o, "after")
    if mode == "fixed":
        # a FIXED pull creates keys too, so it refuses repeats as well
        dup = np.array([base[1], base[2], base[2]], np.uint64)
        with pytest.raises(capi.PskvError) as e:
            t.pull(dup, np.zeros(dup.size * k, np.float32))
        assert e.value.code == capi.EINVAL
        _check_dump(t, o, "after a refused pull")


@pytest.mark.parametrize("memkind", ["device", "host"])
@pytest.mark.parametrize("mode", ["scalar", "fixed", "varlen"])
def test_pushpull_with_too_small_a_buffer_applies_its_push_once(capi, orc, dev, mode, memkind):
    """A push+pull whose response does not fit answers PSKV_ESIZE_MISMATCH with the needed size; its
    push half has been applied (exactly once), so the caller repeats only the pull. This is what the
    second attempt of GpuKVHandle relies on."""
    import torch
    announce("pushpull_too_small", mode, memkind)
    rng = np.random.default_rng(17)
    m = {"scalar": capi.MODE_SCALAR, "fixed": capi.MODE_FIXED, "varlen": capi.MODE_VARLEN}[mode]
    om = {"scalar": orc.MODE_SCALAR, "fixed": orc.MODE_FIXED, "varlen": orc.MODE_VARLEN}[mode]
    t = capi.Table(m, initial_capacity=16)
    o = orc.Store(om)
    n = 3000
    keys = unique_keys(rng, n)
    lens = rng.choice(np.array([0, 4, 8, 12], np.int32), size=n).astype(np.int32) if mode == "varlen" else None
    nvals = {"scalar": n, "fixed": 4 * n, "varlen": int(lens.sum()) if lens is not None else 0}[mode]

    def as_mem(a):
        if a is None:
            return None
        return to_dev(a, dev) if memkind == "device" else a

    for rep in range(3):
        vals = rng.normal(0, 1, size=nvals).astype(np.float32)
        want, want_lens = o.pushpull(keys, vals, lens)
        small_np = np.zeros(max(nvals // 2, 1), np.float32)
        small = as_mem(small_np)
        out_lens = as_mem(np.zeros(n, np.int32)) if mode == "varlen" else None
        with pytest.raises(capi.PskvError) as e:
            t.pushpull(as_mem(keys), as_mem(vals), small, as_mem(lens), out_lens)
        assert e.value.code == capi.ESIZE_MISMATCH
        assert t.last_out_nvals == nvals
        t.sync()
        got = as_mem(np.zeros(nvals, np.float32))
        got_lens = as_mem(np.zeros(n, np.int32)) if mode == "varlen" else None
        assert t.pull(as_mem(keys), got, got_lens) == nvals
        t.sync()
        assert_bits_equal(from_dev(got) if memkind == "device" else got, want, "pull after refused pushpull %d" % rep)
        if mode == "varlen":
            assert np.array_equal(from_dev(got_lens) if memkind == "device" else got_lens, want_lens)
    _check_dump(t, o, "pushpull too small")


@pytest.mark.parametrize("memkind", ["device", "host"])
def test_scalar_key_cache_at_its_real_size(capi, orc, dev, memkind):
    """The stable-key-set path of SCALAR tables with its default threshold: 300,000 keys pushed again
    and again (the third push on is served from the request-ordered value array, 128 bits per lane),
    pulled into aligned and unaligned buffers, then other keys (which must find every slot up to date),
    a shorter request, and the first keys again."""
    import torch
    announce("scalar_key_cache_large", memkind)
    rng = np.random.default_rng(23)
    n = 300000
    keys = unique_keys(rng, n)
    other = unique_keys(rng, n)
    other[: n // 2] = keys[: n // 2]  # half of them shared with the cached set
    other = np.unique(other)
    t = capi.Table(capi.MODE_SCALAR, initial_capacity=16)
    o = orc.Store(orc.MODE_SCALAR)

    def mem(a):
        return to_dev(a, dev) if memkind == "device" else a

    def push(k):
        v = rng.normal(0, 1, size=k.size).astype(np.float32)
        t.push(mem(k), mem(v))
        o.push(k, v)

    def pull(k, shift=0):
        want, _ = o.pull(k)
        if memkind == "device":
            buf = torch.full((k.size + 8,), 7.0, dtype=torch.float32, device=dev)
            out = buf[shift:shift + k.size]
            torch.cuda.synchronize()
            dk = to_dev(k, dev)  # (kept until the wait: the call only enqueues)
            torch.cuda.synchronize()
            t.pull_raw(dk.data_ptr(), k.size, out.data_ptr(), k.size)
            t.sync()
            got = from_dev(out)
        else:
            buf = np.full(k.size + 8, 7.0, np.float32)
            got = buf[shift:shift + k.size]
            t.pull(k, got)
        assert_bits_equal(got, want, "pull shift %d" % shift)

    for _ in range(5):
        push(keys)
    pull(keys)
    pull(keys, shift=1)          # a response buffer that is not 16-byte aligned
    push(keys)
    push(other)                  # other keys: the slots must have caught up first
    pull(other)
    push(keys[:200000])          # a different size
    for _ in range(3):
        push(keys)
    out_np, _ = o.pushpull(keys, np.ones(n, np.float32))
    if memkind == "device":
        out = torch.zeros(n, dtype=torch.float32, device=dev)
        t.pushpull(to_dev(keys, dev), to_dev(np.ones(n, np.float32), dev), out)
        t.sync()
        assert_bits_equal(from_dev(out), out_np, "pushpull")
    else:
        out = np.zeros(n, np.float32)
        t.pushpull(keys, np.ones(n, np.float32), out)
        assert_bits_equal(out, out_np, "pushpull")
    t.sync()
    _check_dump(t, o, "scalar key cache")


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_scalar_key_cache_across_its_default_threshold(capi, orc, dev, seed):
    """Requests of 131,072 keys and more may use the SCALAR key cache, smaller ones never do. Random
    sequences over key sets of 131,071, 131,072 and 140,000 keys (nested, so that a request below
    the threshold changes values that the cache holds for a set above it) and a set of other keys,
    pushes and pulls, device-resident and without a wait between requests: every pull against the
    oracle, the dump at the end."""
    import torch
    announce("scalar_cache_threshold", seed)
    rng = np.random.default_rng(400 + seed)
    big = unique_keys(rng, 140000)
    sets = {"below": big[:131071].copy(), "at": big[:131072].copy(), "above": big,
            "other": unique_keys(rng, 135000)}
    names = ["above", "above", "at", "below", "above", "other", "at"]
    t = capi.Table(capi.MODE_SCALAR, initial_capacity=1 << 18)
    o = orc.Store(orc.MODE_SCALAR)
    checks = []
    for step in range(36):
        name = names[int(rng.integers(0, len(names)))]
        keys = sets[name]
        if rng.random() < 0.6:
            vals = rng.normal(0, 1, size=keys.size).astype(np.float32)
            t.push(to_dev(keys, dev), to_dev(vals, dev))
            o.push(keys, vals)
        else:
            out = torch.full((keys.size,), 7.0, dtype=torch.float32, device=dev)
            t.pull(to_dev(keys, dev), out)
            checks.append((step, name, out, o.pull(keys)[0]))
    t.sync()
    for step, name, out, want in checks:
        assert_bits_equal(from_dev(out), want, "pull of %s at step %d" % (name, step))
    _check_dump(t, o, "across the threshold")


@pytest.mark.parametrize("mode", ["scalar", "fixed", "varlen"])
def test_large_host_requests_travel_piece_by_piece(capi, orc, dev, mode):
    """Host-resident requests of tens of megabytes go through the ring of pinned pieces (8 MiB each):
    copy into the ring, transfer and row kernels overlap piece by piece, in both directions. Sizes that
    are not multiples of a piece, a row length that is not a multiple of four, push, pull and push+pull."""
    announce("large_host_requests", mode)
    rng = np.random.default_rng(31)
    if mode == "scalar":
        n, k = 3000017, 1
        lens = None
    elif mode == "fixed":
        n, k = 1999, 12289  # 98 MB per request, rows that are no multiple of 16 bytes
        lens = None
    else:
        n = 250001
        lens = rng.choice(np.array([0, 8, 16, 64, 128, 300], np.int32), size=n).astype(np.int32)
        k = 0
    nvals = n * k if lens is None else int(lens.sum())
    m = {"scalar": capi.MODE_SCALAR, "fixed": capi.MODE_FIXED, "varlen": capi.MODE_VARLEN}[mode]
    om = {"scalar": orc.MODE_SCALAR, "fixed": orc.MODE_FIXED, "varlen": orc.MODE_VARLEN}[mode]
    t = capi.Table(m, initial_capacity=16)
    o = orc.Store(om)
    keys = unique_keys(rng, n)
    for rep in range(2):
        vals = rng.normal(0, 1, size=nvals).astype(np.float32)
        t.push(keys, vals, lens)
        o.push(keys, vals, lens)
    want, want_lens = o.pull(keys)
    got = np.full(nvals, 7.0, np.float32)
    got_lens = np.full(n, -1, np.int32) if mode == "varlen" else None
    assert t.pull(keys, got, got_lens) == nvals
    assert_bits_equal(got, want, "pull")
    if mode == "varlen":
        assert np.array_equal(got_lens, want_lens)
    vals = rng.normal(0, 1, size=nvals).astype(np.float32)
    want, _ = o.pushpull(keys, vals, lens)
    got = np.full(nvals, 7.0, np.float32)
    t.pushpull(keys, vals, got, lens, got_lens)
    assert_bits_equal(got, want, "pushpull")
    # a pull of half the keys plus as many absent ones (FIXED creates them as zero rows while it answers)
    probe = np.unique(np.concatenate([keys[::2], unique_keys(rng, n // 2)]))
    want, want_lens = o.pull(probe)
    got = np.full(want.size, 7.0, np.float32)
    got_lens = np.full(probe.size, -1, np.int32) if mode == "varlen" else None
    assert t.pull(probe, got, got_lens) == want.size
    assert_bits_equal(got, want, "pull of other keys")
    assert t.size() == o.size()


@pytest.mark.parametrize("memkind", ["device", "host"])
def test_pull_right_behind_a_push_compares_key_by_key(capi, orc, dev, memkind, small_scalar_cache):
    """A worker that pushes gradients and pulls the weights of the same keys (tests/test_kv_app.cc:27-41)
    shows as pulls right behind pushes of their size. Once pushes record themselves, such a pull is
    answered from the recorded values wherever a key sits at its recorded position and through the
    slots elsewhere: pulls of the pushed keys, of keys that differ in a few places (some absent from
    the store, which a pull creates), of a sorted request that repeats a key, and of 2^64-1."""
    import torch
    announce("pull_behind_push", memkind)
    rng = np.random.default_rng(77)
    n = 1500
    t = capi.Table(capi.MODE_SCALAR, initial_capacity=16)
    o = orc.Store(orc.MODE_SCALAR)

    def mem(a):
        return to_dev(a, dev) if memkind == "device" else a

    def push(k):
        v = rng.normal(0, 1, size=k.size).astype(np.float32)
        t.push(mem(k), mem(v))
        o.push(k, v)

    def pull(k, what):
        want, _ = o.pull(k)
        if memkind == "device":
            out = torch.full((k.size,), 7.0, dtype=torch.float32, device=dev)
            t.pull(to_dev(k, dev), out)
            t.sync()
            got = from_dev(out)
        else:
            got = np.full(k.size, 7.0, np.float32)
            t.pull(k, got)
        assert_bits_equal(got, want, what)

    for step in range(4):  # fresh keys every step, as in a sparse model that keeps growing
        k = unique_keys(rng, n)
        push(k)
        pull(k, "same keys, step %d" % step)
    k = unique_keys(rng, n)
    push(k)
    other = k.copy()
    other[10:20] = k[10:20] + np.uint64(1)  # absent keys (a pull creates them), still sorted
    other[700] = k[701]                     # sorted repeats: k[701] twice within four keys,
    other[703] = k[704]                     # k[704] twice across two lanes' keys
    other[1499] = k[1498]                   # and the last key twice
    assert np.all(other[1:] >= other[:-1])
    pull(other, "keys that differ in a few places")
    pull(k, "the pushed keys after all")
    k2 = unique_keys(rng, n)
    k2[-1] = np.uint64(2**64 - 1)
    push(k2)
    pull(k2, "with the largest key")
    shifted = np.sort(np.concatenate([k2[1:], unique_keys(rng, 1)]))
    push(k2)
    pull(shifted, "every position holds another key")
    for step in range(3):
        k = unique_keys(rng, n)
        push(k)
        pull(k, "same keys again, step %d" % step)
    t.sync()
    _check_dump(t, o, "pull behind push")
    t.close()


@pytest.mark.parametrize("mode", ["fixed", "varlen"])
def test_other_rows_in_every_batch(capi, orc, dev, mode):
    """An embedding table's requests: batches of one size that name other rows every time, each pulled and
    then pushed by the worker. The pulls' comparisons with the cached keys keep failing and are skipped
    for longer and longer spells, the pushes repeat their pull's keys; then the same batch comes several
    times in a row (comparisons resume and hit), then other batches again. Every pull and the final store
    against the oracle, requests queued without a wait in between."""
    import torch
    announce("other_rows_in_every_batch", mode)
    rng = np.random.default_rng(31)
    n, universe, k = 700, 5000, 8
    all_keys = unique_keys(rng, universe)
    lens_of = rng.choice([4, 8, 12, 40], size=universe).astype(np.int32)
    m = capi.MODE_FIXED if mode == "fixed" else capi.MODE_VARLEN
    t = capi.Table(m, initial_capacity=2 * universe, row_len=k if mode == "fixed" else 0)
    o = orc.Store(orc.MODE_FIXED if mode == "fixed" else orc.MODE_VARLEN, k if mode == "fixed" else 0)
    held, checks = [], []
    for step in range(70):
        if step in range(40, 46):
            idx = np.arange(100, 100 + n)  # the same batch six times
        else:
            idx = np.sort(rng.choice(universe, size=n, replace=False))
        keys = all_keys[idx]
        lens = lens_of[idx] if mode == "varlen" else None
        nvals = int(lens.sum()) if mode == "varlen" else n * k
        grad = rng.integers(-8, 8, size=nvals).astype(np.float32)
        dk, dg = to_dev(keys, dev), to_dev(grad, dev)
        dl = to_dev(lens, dev) if mode == "varlen" else None
        want, want_lens = o.pull(keys)
        out = torch.full((max(nvals, 1),), 7.0, dtype=torch.float32, device=dev)
        out_lens = torch.full((n,), -1, dtype=torch.int32, device=dev)
        torch.cuda.synchronize()
        t.pull_raw(dk.data_ptr(), n, out.data_ptr(), out.numel(), out_lens.data_ptr() if mode == "varlen" else None)
        t.push_raw(dk.data_ptr(), n, dg.data_ptr(), nvals, dl.data_ptr() if mode == "varlen" else None,
                   n if mode == "varlen" else 0)
        o.push(keys, grad, lens)
        held.append((dk, dg, dl))
        checks.append((step, out, out_lens, want, want_lens))
        if step % 9 == 8:  # now and then the worker waits
            t.sync()
    t.sync()
    for step, out, out_lens, want, want_lens in checks:
        assert_bits_equal(from_dev(out)[:want.size], want, "pull of step %d" % step)
        if mode == "varlen":
            assert np.array_equal(from_dev(out_lens), want_lens), "lens of step %d" % step
    _check_dump(t, o, "other rows in every batch")
    t.close()


def test_scalar_key_cache_written_back_at_scale(capi, orc, dev):
    """1.5M keys pushed four times (the values then live in the request-ordered array, ahead of the
    slots), then other keys: the write-back to the slots, whose launch strides over the keys with a
    bounded number of workgroups, has to bring every slot up to date first. Whole store against the
    oracle."""
    announce("scalar_key_cache_write_back")
    rng = np.random.default_rng(41)
    n = 1500000
    keys = unique_keys(rng, n)
    other = unique_keys(rng, 200000)
    t = capi.Table(capi.MODE_SCALAR, initial_capacity=4 * n)
    o = orc.Store(orc.MODE_SCALAR)
    dk = to_dev(keys, dev)
    for _ in range(4):
        v = rng.normal(0, 1, size=n).astype(np.float32)
        t.push(dk, to_dev(v, dev))
        o.push(keys, v)
    v = rng.normal(0, 1, size=other.size).astype(np.float32)
    t.push(to_dev(other, dev), to_dev(v, dev))
    o.push(other, v)
    t.sync()
    _check_dump(t, o, "write-back at scale")
    t.close()
