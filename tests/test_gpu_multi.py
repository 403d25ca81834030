"""The multi-table entry points (pskv_push_multi / pskv_pull_multi / pskv_sync_multi): all key
ranges of a sliced request served by one launch per pipeline step. Bar: the result of S
single-table calls, i.e. bit-exact against the CPU oracle (one oracle store serves all ranges: they
are disjoint)."""
import numpy as np
import pytest

from conftest import announce
from helpers import assert_bits_equal, covered_limit, from_dev, to_dev, unique_keys

pytestmark = pytest.mark.gpu

MODES = {"scalar": 0, "fixed": 1, "varlen": 2}


def _slice(capi, dk, rb, re, dl=None, nvals=0):
    pos, vpos, used = capi.slice_keys(dk, rb, re, lens=dl, nvals=nvals)
    return pos, vpos


def _dump_all(group):
    ks, ls, vs = [], [], []
    for t in group.tables:
        k, l, v = t.dump()
        ks.append(k), ls.append(l), vs.append(v)
    return np.concatenate(ks), np.concatenate(ls), np.concatenate(vs)


def _check_dump(group, o, what):
    gk, gl, gv = _dump_all(group)  # tables in range order and sorted inside: sorted overall
    ok, ol, ov = o.dump()
    assert np.array_equal(gk, ok), what + ": stored keys differ"
    assert np.array_equal(gl, ol), what + ": stored lens differ"
    assert_bits_equal(gv, ov, what + " dump")


@pytest.mark.parametrize("mode", ["scalar", "fixed", "varlen"])
@pytest.mark.parametrize("S,n", [(1, 3000), (4, 10000), (16, 40000), (37, 20000), (5, 7)])
def test_multi_matches_the_oracle(capi, orc, dev, mode, S, n):
    """Several pushes of changing key sets, a pull of keys of which some are absent; S beyond 16
    (served 16 tables at a time) and requests so small that most slices are empty."""
    import torch
    announce("multi", mode, S, n)
    rng = np.random.default_rng(S * 1000 + n)
    rb, re = capi.server_ranges(S)
    k = 12
    # (FIXED: the row length is given up front, since a table whose range sees no key in the first
    # pushes must still be able to answer a pull)
    g = capi.Group(S, MODES[mode], initial_capacity=16, row_len=k if mode == "fixed" else 0)
    o = orc.Store(MODES[mode], k if mode == "fixed" else 0)
    universe = unique_keys(rng, 2 * n, S)
    len_of = dict(zip(universe.tolist(), rng.choice(np.array([0, 4, 8, 20, 64], np.int32), size=universe.size).tolist()))

    def request(keys):
        lens = np.array([len_of[x] for x in keys.tolist()], np.int32) if mode == "varlen" else None
        nvals = {"scalar": keys.size, "fixed": k * keys.size}.get(mode, int(lens.sum()) if lens is not None else 0)
        return lens, nvals

    for rep in range(4):
        keys = np.sort(rng.choice(universe, size=n, replace=False)) if rep != 2 else keys  # rep 2 repeats rep 1
        lens, nvals = request(keys)
        vals = rng.normal(0, 1, size=nvals).astype(np.float32)
        dk, dv = to_dev(keys, dev), to_dev(vals, dev)
        dl = None if lens is None else to_dev(lens, dev)
        pos, vpos = _slice(capi, dk, rb, re, dl, nvals)
        g.push(dk, pos, dv, vpos, dl)
        o.push(keys, vals, lens)
    g.sync()
    _check_dump(g, o, "after the pushes")

    probe = np.sort(rng.choice(universe, size=n, replace=False))
    want, want_lens = o.pull(probe)
    dk = to_dev(probe, dev)
    pos, _ = _slice(capi, dk, rb, re)
    if mode == "varlen":
        # room per slice = what the oracle says each slice answers, plus slack in some
        lens = want_lens.astype(np.int64)
        off = np.concatenate([[0], np.cumsum(lens)])
        sizes = off[pos.astype(np.int64)[1:]] - off[pos.astype(np.int64)[:-1]]
        room = sizes + (np.arange(S) % 3) * 5
        out_pos = np.concatenate([[0], np.cumsum(room)]).astype(np.uint64)
        out = torch.full((int(out_pos[-1]) + 1,), 7.0, dtype=torch.float32, device=dev)
        out_lens = torch.full((probe.size,), -1, dtype=torch.int32, device=dev)
        got_sizes = g.pull(dk, pos, out, out_pos, out_lens, want_sizes=True)
        g.sync()
        assert np.array_equal(got_sizes.astype(np.int64), sizes)
        assert np.array_equal(from_dev(out_lens), want_lens)
        got = from_dev(out)
        pieces = [got[int(out_pos[s]):int(out_pos[s]) + int(sizes[s])] for s in range(S)]
        assert_bits_equal(np.concatenate(pieces), want, "multi var-len pull")
        # the same without a host round trip
        out2 = torch.full_like(out, 9.0)
        out_lens2 = torch.full_like(out_lens, -1)
        assert g.pull(dk, pos, out2, out_pos, out_lens2) is None
        g.sync()
        got2 = from_dev(out2)
        assert_bits_equal(np.concatenate([got2[int(out_pos[s]):int(out_pos[s]) + int(sizes[s])] for s in range(S)]),
                          want, "multi var-len async pull")
        assert np.array_equal(from_dev(out_lens2), want_lens)
    else:
        width = 1 if mode == "scalar" else k
        out = torch.full((probe.size * width,), 7.0, dtype=torch.float32, device=dev)
        got_sizes = g.pull(dk, pos, out, want_sizes=True)
        g.sync()
        assert np.array_equal(got_sizes.astype(np.int64), np.diff(pos.astype(np.int64)) * width)
        assert_bits_equal(from_dev(out), want, "multi pull")
    _check_dump(g, o, "after the pull")  # SCALAR and FIXED pulls create the absent keys
    g.close()


@pytest.mark.parametrize("mode", ["scalar", "fixed", "varlen"])
@pytest.mark.parametrize("S,n", [(4, 10000), (19, 30000), (3, 300000)])
def test_pushpull_multi_matches_the_oracle(capi, orc, dev, mode, S, n):
    """One request with both halves over all slices (KVWorker::PushPull through kv_app.h:451-459):
    per key the push first, then the value read back; keys the store has never seen among them; the
    third request repeats the second's keys."""
    import torch
    announce("pushpull_multi", mode, S, n)
    rng = np.random.default_rng(S + n)
    rb, re = capi.server_ranges(S)
    k = 12
    g = capi.Group(S, MODES[mode], initial_capacity=16, row_len=k if mode == "fixed" else 0)
    o = orc.Store(MODES[mode], k if mode == "fixed" else 0)
    universe = unique_keys(rng, 2 * n, S)
    len_of = dict(zip(universe.tolist(), rng.choice(np.array([0, 4, 8, 20, 64], np.int32), size=universe.size).tolist()))
    keys = None
    for rep in range(4):
        if rep != 2:
            keys = np.sort(rng.choice(universe, size=n, replace=False))
        lens = np.array([len_of[x] for x in keys.tolist()], np.int32) if mode == "varlen" else None
        nvals = {"scalar": n, "fixed": k * n}.get(mode, int(lens.sum()) if lens is not None else 0)
        vals = rng.normal(0, 1, size=nvals).astype(np.float32)
        dk, dv = to_dev(keys, dev), to_dev(vals, dev)
        dl = None if lens is None else to_dev(lens, dev)
        pos, vpos = _slice(capi, dk, rb, re, dl, nvals)
        out = torch.full((nvals + 4,), 7.0, dtype=torch.float32, device=dev)
        out_lens = torch.full((n,), -1, dtype=torch.int32, device=dev) if mode == "varlen" else None
        sizes = g.pushpull(dk, pos, dv, vpos, out, dl, vpos, out_lens, want_sizes=True)
        rc, want, want_lens, _ = o.handle(True, True, keys, vals, lens)
        assert rc == 0
        g.sync()
        assert np.array_equal(sizes.astype(np.int64), np.diff(vpos.astype(np.int64)))
        assert_bits_equal(from_dev(out)[:nvals], want, "push+pull %d" % rep)
        if mode == "varlen":
            assert np.array_equal(from_dev(out_lens), want_lens)
    _check_dump(g, o, "after the push+pulls")
    g.close()


def test_multi_equals_single_table_calls(capi, dev):
    """The same requests through pskv_push_multi and through one pskv_push per table leave
    identical stores, key for key and bit for bit (var-len rows of mixed lengths)."""
    announce("multi_vs_single")
    rng = np.random.default_rng(3)
    S, n = 8, 30000
    rb, re = capi.server_ranges(S)
    keys = unique_keys(rng, n, S)
    lens = rng.choice(np.array([8, 16, 32, 64, 128], np.int32), size=n).astype(np.int32)
    nvals = int(lens.sum())
    dk, dl = to_dev(keys, dev), to_dev(lens, dev)
    pos, vpos = _slice(capi, dk, rb, re, dl, nvals)
    g = capi.Group(S, capi.MODE_VARLEN, initial_capacity=16)
    singles = [capi.Table(capi.MODE_VARLEN, initial_capacity=16) for _ in range(S)]
    p, vp = pos.astype(np.int64), vpos.astype(np.int64)
    for rep in range(3):
        vals = rng.normal(0, 0.1, size=nvals).astype(np.float32)
        dv = to_dev(vals, dev)
        g.push(dk, pos, dv, vpos, dl)
        for s in range(S):
            singles[s].push(dk[p[s]:p[s + 1]], dv[vp[s]:vp[s + 1]], dl[p[s]:p[s + 1]])
        g.sync()
    for s in range(S):
        a, b = g.tables[s].dump(), singles[s].dump()
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
        assert_bits_equal(a[2], b[2], "table %d" % s)


def test_multi_misuse_is_a_status_code(capi, dev):
    import torch
    announce("multi_misuse")
    S = 3
    rb, re = capi.server_ranges(S)
    rng = np.random.default_rng(8)
    keys = unique_keys(rng, 300, S)
    dk = to_dev(keys, dev)
    dv = to_dev(np.ones(keys.size, np.float32), dev)
    pos, vpos = _slice(capi, dk, rb, re, None, keys.size)
    # tables with streams of their own cannot share a launch
    loose = [capi.Table(capi.MODE_SCALAR) for _ in range(S)]
    arr = (capi.ctypes.c_void_p * S)(*[t._h for t in loose])
    rc = capi.load().pskv_push_multi(arr, S, dk.data_ptr(), pos.ctypes.data, dv.data_ptr(), vpos.ctypes.data,
                                     None, capi.MEM_DEVICE)
    assert rc == capi.EINVAL and b"stream" in capi.load().pskv_last_error()
    g = capi.Group(S, capi.MODE_SCALAR)
    # host buffers go table by table
    rc = capi.load().pskv_push_multi(g._arr, S, keys.ctypes.data, pos.ctypes.data, dv.data_ptr(), vpos.ctypes.data,
                                     None, capi.MEM_HOST)
    assert rc == capi.EINVAL
    # values that do not match the keys of one slice (kv_app.h:447): nothing is applied anywhere
    bad = vpos.copy()
    bad[1] += np.uint64(1)
    with pytest.raises(capi.PskvError) as e:
        g.push(dk, pos, dv, bad)
    assert e.value.code == capi.ESIZE_MISMATCH
    g.sync()
    assert g.size() == (0, 0)
    # a pull whose slice has too little room
    out = torch.zeros(keys.size, dtype=torch.float32, device=dev)
    small = pos.copy()
    small[1:] -= np.uint64(1)
    with pytest.raises(capi.PskvError) as e:
        g.pull(dk, pos, out, small)
    assert e.value.code == capi.ESIZE_MISMATCH
    assert g.size() == (0, 0)
    # a var-len push with a changed length in ONE table is reported by the group's sync, once
    gv = capi.Group(S, capi.MODE_VARLEN)
    lens = np.full(keys.size, 4, np.int32)
    dl = to_dev(lens, dev)
    dv4 = to_dev(np.ones(keys.size * 4, np.float32), dev)
    pos, vpos = _slice(capi, dk, rb, re, dl, keys.size * 4)
    gv.push(dk, pos, dv4, vpos, dl)
    gv.sync()
    lens2 = lens.copy()
    lens2[5] = 8
    dl2 = to_dev(lens2, dev)
    dv5 = to_dev(np.ones(int(lens2.sum()), np.float32), dev)
    pos2, vpos2 = _slice(capi, dk, rb, re, dl2, int(lens2.sum()))
    gv.push(dk, pos2, dv5, vpos2, dl2)
    with pytest.raises(capi.PskvError) as e:
        gv.sync()
    assert e.value.code == capi.ELEN_CHANGED
    gv.sync()
    # the other tables took their slices: only table 0 refused
    sizes = [t.size()[0] for t in gv.tables]
    assert sum(sizes) == keys.size


def test_multi_scalar_tables_with_repeating_key_sets(capi, orc, dev, monkeypatch):
    """SCALAR tables of a group whose requests repeat their key set: every table takes its own
    decision (serve from its request-ordered value array, or go through the slots) inside the one
    launch that serves them all."""
    import torch
    announce("multi_scalar_repeats")
    monkeypatch.setenv("PSKV_SCALAR_CACHE_MIN_KEYS", "64")
    rng = np.random.default_rng(77)
    S, n = 6, 30000
    rb, re = capi.server_ranges(S)
    g = capi.Group(S, capi.MODE_SCALAR, initial_capacity=16)
    o = orc.Store(orc.MODE_SCALAR)
    a = unique_keys(rng, n, S)
    b = a.copy()
    # b differs from a in the keys of two ranges only: the other tables keep serving from their cache
    lim = covered_limit(S) // S
    for s in (1, 4):
        m = (b >= s * lim) & (b < (s + 1) * lim)
        b[m] = np.sort(rng.integers(s * lim, (s + 1) * lim, size=int(m.sum()), dtype=np.uint64))
    b = np.unique(b)
    for name in "a a a a b a a b b a".split():
        keys = a if name == "a" else b
        vals = rng.normal(0, 1, size=keys.size).astype(np.float32)
        dk, dv = to_dev(keys, dev), to_dev(vals, dev)
        pos, vpos = _slice(capi, dk, rb, re, None, keys.size)
        g.push(dk, pos, dv, vpos)
        o.push(keys, vals)
        out = torch.full((keys.size,), 7.0, dtype=torch.float32, device=dev)
        g.pull(dk, pos, out)
        g.sync()
        assert_bits_equal(from_dev(out), o.pull(keys)[0], "pull after push of " + name)
    _check_dump(g, o, "multi scalar repeats")
    g.close()
