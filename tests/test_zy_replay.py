"""Recorded requests (pskv_replay_record / pskv_replay_run): a request that repeats, kept as a HIP
graph and applied again with one launch. Bar: every run leaves what the same request through
pskv_push_multi / pskv_pull_multi leaves, i.e. bit-exact against the CPU oracle, run after run, with
the program's own eager work and waits between the runs; a run whose keys have changed applies and
answers nothing and is reported; any other request on the tables ends the recording's life."""
import numpy as np
import pytest

from conftest import announce
from helpers import assert_bits_equal, from_dev, to_dev, unique_keys

pytestmark = pytest.mark.gpu

MODES = {"scalar": 0, "fixed": 1, "varlen": 2}
K = 12


def _request(rng, mode, keys):
    lens = rng.choice(np.array([0, 4, 8, 20, 64], np.int32), size=keys.size).astype(np.int32) if mode == "varlen" else None
    nvals = {"scalar": keys.size, "fixed": K * keys.size}.get(mode, int(lens.sum()) if lens is not None else 0)
    return lens, nvals


def _dump_all(group):
    ks, ls, vs = [], [], []
    for t in group.tables:
        k, l, v = t.dump()
        ks.append(k), ls.append(l), vs.append(v)
    return np.concatenate(ks), np.concatenate(ls), np.concatenate(vs)


def _check_dump(group, o, what):
    gk, gl, gv = _dump_all(group)
    ok, ol, ov = o.dump()
    assert np.array_equal(gk, ok), what + ": stored keys differ"
    assert np.array_equal(gl, ol), what + ": stored lens differ"
    assert_bits_equal(gv, ov, what + " dump")


class _Step:
    """One request (push, pull, or the one behind the other) on device buffers that stay where they are."""

    def __init__(self, capi, dev, rng, mode, S, keys, lens, nvals):
        import torch
        self.capi, self.mode, self.S = capi, mode, S
        self.keys, self.lens, self.nvals = keys, lens, nvals
        rb, re = capi.server_ranges(S)
        self.dk = to_dev(keys, dev)
        self.dl = None if lens is None else to_dev(lens, dev)
        self.pos, self.vpos, _ = capi.slice_keys(self.dk, rb, re, lens=self.dl, nvals=nvals)
        self.dv = torch.zeros(max(nvals, 1), dtype=torch.float32, device=dev)[:nvals]
        self.out = torch.full((nvals + 8,), 7.0, dtype=torch.float32, device=dev)
        self.out_lens = torch.full((keys.size,), -1, dtype=torch.int32, device=dev) if mode == "varlen" else None
        # the response of slice s starts where its values start in the request
        self.out_pos = self.vpos.copy()

    def set_vals(self, vals):
        import torch
        self.dv.copy_(torch.from_numpy(vals))
        self.out.fill_(7.0)
        if self.out_lens is not None:
            self.out_lens.fill_(-1)
        torch.cuda.synchronize()

    def answered(self):
        return from_dev(self.out)[:self.nvals]


@pytest.mark.parametrize("mode", ["scalar", "fixed", "varlen"])
@pytest.mark.parametrize("S,n", [(4, 400000), (1, 1000), (16, 40000), (37, 9000)])
@pytest.mark.parametrize("what", ["push+pull", "push", "pull"])
@pytest.mark.parametrize("how", ["graph", "launches"])
def test_replays_equal_the_oracle(capi, orc, dev, mode, S, n, what, how):
    import torch
    announce("replay", mode, S, n, what, how)
    rng = np.random.default_rng(S * 7 + n + len(what))
    g = capi.Group(S, MODES[mode], initial_capacity=16, row_len=K if mode == "fixed" else 0)
    o = orc.Store(MODES[mode], K if mode == "fixed" else 0)
    keys = unique_keys(rng, n, S)
    lens, nvals = _request(rng, mode, keys)
    st = _Step(capi, dev, rng, mode, S, keys, lens, nvals)
    # something is in the tables already, under other keys and under these
    other = unique_keys(rng, n // 2 + 1, S)
    ol, onv = _request(rng, mode, other)
    ov = rng.normal(0, 1, size=onv).astype(np.float32)
    dko, dvo = to_dev(other, dev), to_dev(ov, dev)
    dlo = None if ol is None else to_dev(ol, dev)
    rb, re = capi.server_ranges(S)
    p, vp, _ = capi.slice_keys(dko, rb, re, lens=dlo, nvals=onv)
    g.push(dko, p, dvo, vp, dlo)
    o.push(other, ov, ol)
    first = rng.normal(0, 1, size=nvals).astype(np.float32)
    if what == "pull":  # a pull of keys that nobody pushed answers zeros (and nothing in var-len mode)
        st.set_vals(first)
        g.push(st.dk, st.pos, st.dv, st.vpos, st.dl)
        o.push(keys, first, lens)
        g.sync()
    flags = {"push+pull": capi.REPLAY_PUSH | capi.REPLAY_PULL, "push": capi.REPLAY_PUSH, "pull": capi.REPLAY_PULL}[what]
    if how == "launches":
        flags |= capi.REPLAY_LAUNCHES

    def reference(vals):
        if "push" in what:
            o.push(keys, vals, lens)
        if "pull" in what:
            return o.pull(keys)
        return None, None

    def check(tag):
        if "pull" not in what:
            return
        want, want_lens = expect
        assert_bits_equal(st.answered(), want, tag)
        if mode == "varlen":
            assert np.array_equal(from_dev(st.out_lens), want_lens), tag

    vals = rng.normal(0, 1, size=nvals).astype(np.float32)
    st.set_vals(vals)
    rec = g.record(flags, st.dk, st.pos, st.dv, st.vpos, st.dl, st.out if "pull" in what else None,
                   st.out_pos if "pull" in what else None, st.out_lens if "pull" in what else None)
    expect = reference(vals)  # recording a request serves it once
    g.sync()
    check("the recording run")
    for rep in range(6):
        vals = rng.normal(0, 1, size=nvals).astype(np.float32)
        st.set_vals(vals)
        rec.run()
        if rep % 2 == 0:
            rec.run()  # two runs in a row without a wait between them
            reference(vals)
        expect = reference(vals)
        g.sync()
        check("run %d" % rep)
        if rep == 3:
            # eager work of the program's own between the runs: sizes (a wait and a read-back)
            assert g.size()[0] == o.size()[0]
            torch.cuda.synchronize()
    rec.close()
    _check_dump(g, o, "after the replays")
    g.close()


@pytest.mark.parametrize("mode", ["scalar", "fixed", "varlen"])
@pytest.mark.parametrize("how", [0, 4])  # a graph / the launches one by one (PSKV_REPLAY_LAUNCHES)
def test_a_replay_whose_keys_have_changed_applies_nothing(capi, orc, dev, mode, how):
    import torch
    announce("replay_changed_keys", mode, how)
    rng = np.random.default_rng(11)
    S, n = 4, 50000
    g = capi.Group(S, MODES[mode], initial_capacity=16, row_len=K if mode == "fixed" else 0)
    o = orc.Store(MODES[mode], K if mode == "fixed" else 0)
    keys = unique_keys(rng, n, S)
    lens, nvals = _request(rng, mode, keys)
    st = _Step(capi, dev, rng, mode, S, keys, lens, nvals)
    vals = rng.normal(0, 1, size=nvals).astype(np.float32)
    st.set_vals(vals)
    rec = g.record(capi.REPLAY_PUSH | capi.REPLAY_PULL | how, st.dk, st.pos, st.dv, st.vpos, st.dl, st.out, st.out_pos,
                   st.out_lens)
    o.push(keys, vals, lens)
    g.sync()
    rec.run()
    o.push(keys, vals, lens)
    g.sync()
    # one key of the third slice becomes another (still sorted, still inside its range)
    at = int(st.pos[2]) + 5
    saved = st.dk[at].clone()
    st.dk[at] = st.dk[at] + 1
    assert int(st.dk[at]) < int(st.dk[at + 1])
    st.set_vals(vals)
    rec.run()
    with pytest.raises(capi.PskvError) as e:
        g.sync()
    assert e.value.code == capi.ESTALE
    # the other slices were served, the third neither applied nor answered
    p, vp = st.pos.astype(np.int64), st.vpos.astype(np.int64)
    mask = np.ones(n, bool)
    mask[p[2]:p[3]] = False
    if mode == "varlen":
        o.push(keys[mask], np.concatenate([vals[:vp[2]], vals[vp[3]:]]), lens[mask])
    elif mode == "fixed":
        o.push(keys[mask], np.concatenate([vals[:vp[2]], vals[vp[3]:]]), None)
    else:
        o.push(keys[mask], vals[mask], None)
    got = st.answered()
    assert np.all(got[vp[2]:vp[3]] == 7.0)
    st.dk[at] = saved
    torch.cuda.synchronize()
    # with the keys back, the recording serves the request again
    rec.run()
    o.push(keys, vals, lens)
    want, _ = o.pull(keys)
    g.sync()
    assert_bits_equal(st.answered(), want, "after the keys came back")
    rec.close()
    _check_dump(g, o, "changed keys")
    g.close()


@pytest.mark.parametrize("mode", ["scalar", "varlen"])
def test_another_request_ends_a_recording(capi, orc, dev, mode):
    announce("replay_stale", mode)
    rng = np.random.default_rng(5)
    S, n = 3, 20000
    g = capi.Group(S, MODES[mode], initial_capacity=16)
    o = orc.Store(MODES[mode], 0)
    keys = unique_keys(rng, n, S)
    lens, nvals = _request(rng, mode, keys)
    st = _Step(capi, dev, rng, mode, S, keys, lens, nvals)
    vals = rng.normal(0, 1, size=nvals).astype(np.float32)
    st.set_vals(vals)
    rec = g.record(capi.REPLAY_PUSH, st.dk, st.pos, st.dv, st.vpos, st.dl)
    o.push(keys, vals, lens)
    rec.run()
    o.push(keys, vals, lens)
    # an ordinary push of new keys to one table: it may grow, the cache is another request's now
    more = unique_keys(rng, 5000, S)
    more = more[(more >= keys[int(st.pos[1])]) & (more < keys[int(st.pos[2]) - 1])]
    more = np.setdiff1d(more, keys)
    ml, mnv = _request(rng, mode, more)
    mv = rng.normal(0, 1, size=mnv).astype(np.float32)
    g.tables[1].push(to_dev(more, dev), to_dev(mv, dev), None if ml is None else to_dev(ml, dev))
    o.push(more, mv, ml)
    with pytest.raises(capi.PskvError) as e:
        rec.run()
    assert e.value.code == capi.ESTALE
    g.sync()
    rec.close()
    # recorded again, it runs again
    rec = g.record(capi.REPLAY_PUSH, st.dk, st.pos, st.dv, st.vpos, st.dl)
    o.push(keys, vals, lens)
    for _ in range(3):
        rec.run()
        o.push(keys, vals, lens)
    g.sync()
    rec.close()
    _check_dump(g, o, "after the second recording")
    g.close()


@pytest.mark.parametrize("mode", ["scalar", "fixed", "varlen"])
def test_recording_behind_another_key_set_of_the_same_size(capi, orc, dev, mode):
    """The key cache holds a request of the same size but other keys when the recording starts, the
    tables time their launches (a recording must not carry events), and the stream is the caller's."""
    import torch
    announce("replay_same_size", mode)
    rng = np.random.default_rng(23)
    S, n = 4, 300000
    stream = torch.cuda.Stream()
    g = capi.Group(S, MODES[mode], initial_capacity=16, row_len=K if mode == "fixed" else 0, stream=stream.cuda_stream)
    o = orc.Store(MODES[mode], K if mode == "fixed" else 0)
    for t in g.tables:
        t.prof_enable(True)
    for seed in (1, 2):
        keys = unique_keys(np.random.default_rng(seed), n, S)
        lens, nvals = _request(rng, mode, keys)
        st = _Step(capi, dev, rng, mode, S, keys, lens, nvals)
        vals = rng.normal(0, 1, size=nvals).astype(np.float32)
        st.set_vals(vals)
        if seed == 1:  # twice, so that the second push is served from the key cache
            for _ in range(2):
                g.push(st.dk, st.pos, st.dv, st.vpos, st.dl)
                o.push(keys, vals, lens)
            g.sync()
            continue
        rec = g.record(capi.REPLAY_PUSH | capi.REPLAY_PULL, st.dk, st.pos, st.dv, st.vpos, st.dl, st.out, st.out_pos,
                       st.out_lens)
        o.push(keys, vals, lens)
        for rep in range(3):
            vals = rng.normal(0, 1, size=nvals).astype(np.float32)
            st.set_vals(vals)
            rec.run()
            o.push(keys, vals, lens)
            want, want_lens = o.pull(keys)
            g.sync()
            assert_bits_equal(st.answered(), want, "run %d" % rep)
            if mode == "varlen":
                assert np.array_equal(from_dev(st.out_lens), want_lens)
        rec.close()
    _check_dump(g, o, "same size")
    g.close()


def test_replay_misuse_is_a_status_code(capi, dev):
    import torch
    announce("replay_misuse")
    g = capi.Group(2, capi.MODE_SCALAR)
    keys = torch.arange(10, dtype=torch.int64, device=dev)
    vals = torch.ones(10, dtype=torch.float32, device=dev)
    pos = np.array([0, 10, 10], np.uint64)
    for what in (0, 4, 8, 15):
        with pytest.raises(capi.PskvError) as e:
            g.record(what, keys, pos, vals, pos)
        assert e.value.code == capi.EINVAL
    with pytest.raises(capi.PskvError) as e:
        g.record(capi.REPLAY_PUSH, keys, np.array([0, 0, 0], np.uint64), vals, np.array([0, 0, 0], np.uint64))
    assert e.value.code == capi.EINVAL
    with pytest.raises(capi.PskvError) as e:  # values without positions
        g.record(capi.REPLAY_PUSH, keys, pos, vals, None)
    assert e.value.code == capi.EINVAL
    g.sync()
    g.close()
    # a var-len pull leaves no key cache behind: on its own it can only be recorded behind a push of its keys
    g = capi.Group(2, capi.MODE_VARLEN)
    lens = torch.full((10,), 4, dtype=torch.int32, device=dev)
    vals = torch.ones(40, dtype=torch.float32, device=dev)
    out = torch.zeros(40, dtype=torch.float32, device=dev)
    out_lens = torch.zeros(10, dtype=torch.int32, device=dev)
    vpos = np.array([0, 40, 40], np.uint64)
    with pytest.raises(capi.PskvError) as e:
        g.record(capi.REPLAY_PULL, keys, pos, None, None, None, out, vpos, out_lens)
    assert e.value.code == capi.ESTALE and "PSKV_MODE_VARLEN pull" in str(e.value)
    g.push(keys, pos, vals, vpos, lens)
    rec = g.record(capi.REPLAY_PULL, keys, pos, None, None, None, out, vpos, out_lens)
    rec.run()
    g.sync()
    assert torch.equal(out, vals) and torch.equal(out_lens, lens)
    rec.close()
    g.close()
