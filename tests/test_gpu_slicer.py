"""GPU parity of the key-range slicer and of the pull reassembly against the CPU oracle,
through the C ABI. Bar: identical integers and identical error codes."""
import numpy as np
import pytest

from conftest import announce
from helpers import KMAX, assert_bits_equal, covered_limit, from_dev, to_dev, unique_keys

pytestmark = pytest.mark.gpu


def _compare(capi, orc, keys, rb, re, lens, nvals, dev, memkind):
    rc, o_pos, o_vpos, o_used = orc.slice_status(keys, rb, re, lens, nvals)
    k = to_dev(keys, dev) if memkind == "device" else keys
    l = None if lens is None else (to_dev(lens, dev) if memkind == "device" else lens)
    try:
        pos, vpos, used = capi.slice_keys(k, rb, re, lens=l, nvals=nvals)
    except capi.PskvError as e:
        assert e.code == rc, (e.code, rc)
        return rc
    assert rc == 0
    assert np.array_equal(pos, o_pos), (pos, o_pos)
    assert np.array_equal(vpos, o_vpos), (vpos, o_vpos)
    assert np.array_equal(used, o_used)
    return 0


@pytest.mark.parametrize("memkind", ["device", "host"])
@pytest.mark.parametrize("n,S", [(0, 4), (1, 1), (63, 3), (64, 4), (65, 16), (4096, 7), (4097, 64), (5000, 31), (5000, 32),
                                 (100000, 4), (262145, 16), (1000003, 1), (2000000, 16)])
def test_slice_uniform(capi, orc, dev, memkind, n, S):
    announce("slice_uniform", memkind, n, S)
    rng = np.random.default_rng(n + S)
    rb, re = capi.server_ranges(S)
    o_rb, o_re = orc.server_ranges(S)
    assert np.array_equal(rb, o_rb) and np.array_equal(re, o_re)
    keys = unique_keys(rng, n, S) if n else np.zeros(0, np.uint64)
    # no lens, k = 3
    assert _compare(capi, orc, keys, rb, re, None, 3 * n, dev, memkind) == 0
    # lens
    lens = rng.choice(np.array([8, 16, 32, 64, 128], np.int32), size=n).astype(np.int32)
    assert _compare(capi, orc, keys, rb, re, lens, int(lens.sum()), dev, memkind) == 0
    # pull request: no values at all (kv_app.h:151-164)
    assert _compare(capi, orc, keys, rb, re, None, 0, dev, memkind) == 0


@pytest.mark.parametrize("S", [1, 64, 1024])
def test_slice_sixteen_million_keys(capi, dev, S):
    """The largest request of the benchmark configurations (a pull of 16M keys): positions against
    numpy's searchsorted, the lens sums against cumsum, and the invariants of kv_app.h:528-542."""
    announce("slice_16M", S)
    n = 16000000
    rng = np.random.default_rng(16 + S)
    rb, re = capi.server_ranges(S)
    keys = unique_keys(rng, n, S)
    lens = rng.integers(0, 5, size=n).astype(np.int32)
    dk, dl = to_dev(keys, dev), to_dev(lens, dev)
    pos, vpos, used = capi.slice_keys(dk, rb, re, lens=dl, nvals=int(lens.sum()))
    want = np.concatenate([[np.searchsorted(keys, rb[0], side="left")], np.searchsorted(keys, re, side="left")])
    assert np.array_equal(pos.astype(np.int64), want.astype(np.int64))
    assert pos[0] == 0 and pos[-1] == n and np.all(np.diff(pos.astype(np.int64)) >= 0)
    off = np.concatenate([[0], np.cumsum(lens.astype(np.int64))])
    assert np.array_equal(vpos.astype(np.int64), off[pos.astype(np.int64)])
    assert np.array_equal(used.astype(bool), np.diff(pos.astype(np.int64)) > 0)
    pos2, vpos2, _ = capi.slice_keys(dk, rb, re, nvals=2 * n)  # no lens: k = 2
    assert np.array_equal(pos2, pos) and np.array_equal(vpos2.astype(np.int64), 2 * pos.astype(np.int64))


@pytest.mark.parametrize("S", [1, 4, 1024])
def test_slice_sixteen_million_keys_in_host_memory(capi, orc, dev, S):
    """The same request with its keys (and lens) in ordinary host memory, as the worker's slicer
    gets them (kv_app.h:517-572): host-resident keys are searched where they lie, the lens of a
    request this large are added up on the GPU. Positions, value offsets and flags against the oracle."""
    announce("slice_16M_host", S)
    n = 16000000
    rng = np.random.default_rng(61 + S)
    rb, re = capi.server_ranges(S)
    keys = unique_keys(rng, n, S)
    lens = rng.integers(0, 5, size=n).astype(np.int32)
    assert _compare(capi, orc, keys, rb, re, None, 2 * n, dev, "host") == 0
    assert _compare(capi, orc, keys, rb, re, lens, int(lens.sum()), dev, "host") == 0
    # a key past the last range: the reference's CHECK at kv_app.h:542
    bad = keys.copy()
    bad[-1] = np.uint64(KMAX)
    assert _compare(capi, orc, bad, rb, re, None, 2 * n, dev, "host") == capi.EUNCOVERED_KEY


@pytest.mark.parametrize("memkind", ["device", "host"])
def test_slice_skewed_and_edges(capi, orc, dev, memkind):
    """All keys in one range, keys sitting exactly on range boundaries, empty middle slices."""
    announce("slice_skewed", memkind)
    S = 8
    rb, re = capi.server_ranges(S)
    rng = np.random.default_rng(3)
    for s in (0, 3, 7):
        keys = np.unique(rng.integers(int(rb[s]), int(re[s]), size=5000, dtype=np.uint64))
        assert _compare(capi, orc, keys, rb, re, None, 2 * keys.size, dev, memkind) == 0
    edge = np.unique(np.concatenate([rb, re - np.uint64(1), re[:-1], re[:-1] + np.uint64(1)]))
    lens = (np.arange(edge.size) % 5).astype(np.int32)
    assert _compare(capi, orc, edge, rb, re, lens, int(lens.sum()), dev, memkind) == 0
    two = np.array([int(rb[1]) + 5, int(rb[6]) + 5], np.uint64)
    assert _compare(capi, orc, two, rb, re, np.array([3, 4], np.int32), 7, dev, memkind) == 0


@pytest.mark.parametrize("memkind", ["device", "host"])
def test_slice_errors(capi, orc, dev, memkind):
    announce("slice_errors", memkind)
    S = 4
    rb, re = capi.server_ranges(S)
    keys = np.array([0, 1, KMAX // 4 - 1, KMAX // 4, KMAX // 4 * 2 + 5, KMAX - 3], np.uint64)
    # the top keys are covered by no range (kv_app.h:542)
    assert _compare(capi, orc, keys, rb, re, None, 6, dev, memkind) == capi.EUNCOVERED_KEY
    ok = keys.copy()
    ok[-1] = covered_limit(4) - 1
    assert _compare(capi, orc, ok, rb, re, None, 7, dev, memkind) == capi.ESIZE_MISMATCH  # :549
    lens = np.array([1, 0, 3, 2, 5, 1], np.int32)
    assert _compare(capi, orc, ok, rb, re, lens[:5], 12, dev, memkind) == capi.ESIZE_MISMATCH  # :551
    assert _compare(capi, orc, ok, rb, re, lens, 11, dev, memkind) == capi.ESIZE_MISMATCH  # sarray.h:249
    assert _compare(capi, orc, ok, rb, re, lens, 20, dev, memkind) == 0  # trailing values are ignored
    gap_rb = rb.copy()
    gap_rb[2] += np.uint64(1)
    assert _compare(capi, orc, ok, gap_rb, re, None, 6, dev, memkind) == capi.ERANGE_GAP  # :533
    # caller-supplied ranges that start above the first keys: the front keys are skipped and,
    # with lens, the value offsets still start at 0 (kv_app.h:530,546)
    sub_rb, sub_re = rb[1:].copy(), re[1:].copy()
    tail = ok[3:]
    assert _compare(capi, orc, tail, sub_rb, sub_re, lens[3:], 8, dev, memkind) == 0
    # without lens the skipped front keys are simply not sent: pos[0] = 3, pos[S] = n
    assert _compare(capi, orc, ok, sub_rb, sub_re, None, 12, dev, memkind) == 0


def test_slice_threads(capi, orc, dev):
    """KVWorker::Push is thread-safe (kv_app.h:101-104): concurrent slicer calls agree with serial ones."""
    import threading
    announce("slice_threads")
    S = 16
    rb, re = capi.server_ranges(S)
    rng = np.random.default_rng(11)
    work = []
    for i in range(8):
        keys = unique_keys(rng, 20000 + 1000 * i, S)
        lens = rng.integers(0, 50, size=keys.size).astype(np.int32)
        work.append((keys, lens, to_dev(keys, dev), to_dev(lens, dev)))
    results = [None] * len(work)

    def run(i):
        keys, lens, dk, dl = work[i]
        for _ in range(5):
            results[i] = capi.slice_keys(dk, rb, re, lens=dl, nvals=int(lens.sum()))

    threads = [threading.Thread(target=run, args=(i,)) for i in range(len(work))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for i, (keys, lens, _, _) in enumerate(work):
        o_pos, o_vpos, o_used = orc.slice_keys(keys, rb, re, lens, int(lens.sum()))
        assert np.array_equal(results[i][0], o_pos) and np.array_equal(results[i][1], o_vpos)


def test_slice_push_pull_round_trip(capi, orc, dev):
    """Slicer -> one var-len table per range -> pull per range -> reassembly gives back exactly
    what a single oracle store holds (the layout round trip of kv_app.h:562-570 and 663-714)."""
    import torch
    announce("slice_round_trip")
    S = 5
    rng = np.random.default_rng(21)
    rb, re = capi.server_ranges(S)
    keys = unique_keys(rng, 30000, S)
    lens = rng.choice(np.array([0, 4, 8, 12, 100], np.int32), size=keys.size).astype(np.int32)
    nvals = int(lens.sum())
    dk, dl = to_dev(keys, dev), to_dev(lens, dev)
    tables = [capi.Table(capi.MODE_VARLEN, initial_capacity=1024) for _ in range(S)]
    o = orc.Store(orc.MODE_VARLEN)
    pos, vpos, used = capi.slice_keys(dk, rb, re, lens=dl, nvals=nvals)
    pos, vpos = pos.astype(np.int64), vpos.astype(np.int64)
    for rep in range(3):
        vals = rng.normal(0, 0.1, size=nvals).astype(np.float32)
        dv = to_dev(vals, dev)
        for s in range(S):
            if used[s]:
                tables[s].push(dk[pos[s]:pos[s + 1]], dv[vpos[s]:vpos[s + 1]], dl[pos[s]:pos[s + 1]])
        o.push(keys, vals, lens)
    responses = []
    for s in reversed(range(S)):  # responses arrive in any order
        if not used[s]:
            continue
        ks = dk[pos[s]:pos[s + 1]]
        out = torch.empty(int(vpos[s + 1] - vpos[s]), dtype=torch.float32, device=dev)
        out_lens = torch.empty(ks.numel(), dtype=torch.int32, device=dev)
        tables[s].pull(ks, out, out_lens)
        tables[s].sync()
        responses.append((ks, out, out_lens))
    out = torch.empty(nvals, dtype=torch.float32, device=dev)
    out_lens = torch.empty(keys.size, dtype=torch.int32, device=dev)
    assert capi.assemble_pull(dk, responses, out, out_lens) == nvals
    want, want_lens = o.pull(keys)
    assert np.array_equal(from_dev(out_lens), want_lens)
    assert_bits_equal(from_dev(out), want, "round trip")
    # the oracle's reassembly agrees as well
    rc, o_vals, o_lens = orc.assemble_pull(
        keys, [(from_dev(k).view(np.uint64), from_dev(v), from_dev(l)) for k, v, l in responses], True)
    assert rc == 0 and np.array_equal(o_lens, want_lens)
    assert_bits_equal(o_vals, want, "oracle reassembly")


@pytest.mark.parametrize("R", [1, 3, 7])
def test_assemble_pieces_on_any_word_boundary(capi, dev, R):
    """The reassembly copies every slice to its place with one launch; slices of 1, 2, 3, 5... floats
    make sources and destinations start on any 4-byte boundary, and some are shorter than 16 bytes."""
    import torch
    announce("assemble_unaligned", R)
    rng = np.random.default_rng(70 + R)
    n = 5000
    keys = unique_keys(rng, n)
    lens = rng.choice(np.array([0, 1, 2, 3, 5, 7, 33], np.int32), size=n).astype(np.int32)
    cuts = np.sort(rng.choice(np.arange(1, n), size=R - 1, replace=False)) if R > 1 else np.zeros(0, np.int64)
    pos = np.concatenate([[0], cuts, [n]]).astype(np.int64)
    off = np.concatenate([[0], np.cumsum(lens.astype(np.int64))])
    vals = rng.standard_normal(int(off[-1])).astype(np.float32)
    dk = to_dev(keys, dev)
    # every response lives at an odd offset of a larger buffer, so its start is not 16-byte aligned
    responses = []
    for r in range(R):
        a, b = int(pos[r]), int(pos[r + 1])
        pad = int(rng.integers(1, 4))
        vbuf = torch.zeros(int(off[b] - off[a]) + pad, dtype=torch.float32, device=dev)
        vbuf[pad:] = to_dev(vals[off[a]:off[b]], dev)
        lbuf = torch.zeros(b - a + pad, dtype=torch.int32, device=dev)
        lbuf[pad:] = to_dev(lens[a:b], dev)
        responses.append((dk[a:b], vbuf[pad:], lbuf[pad:]))
    order = rng.permutation(R)
    responses = [responses[i] for i in order]
    guard = 3
    out = torch.full((vals.size + 2 * guard,), 7.0, dtype=torch.float32, device=dev)
    out_lens = torch.full((n + 2 * guard,), -1, dtype=torch.int32, device=dev)
    got = capi.assemble_pull(dk, responses, out[guard:guard + vals.size], out_lens[guard:guard + n])
    assert got == vals.size
    o, ol = from_dev(out), from_dev(out_lens)
    assert_bits_equal(o[guard:guard + vals.size], vals, "assembled values")
    assert np.array_equal(ol[guard:guard + n], lens)
    assert np.all(o[:guard] == 7.0) and np.all(o[guard + vals.size:] == 7.0), "wrote outside the response"
    assert np.all(ol[:guard] == -1) and np.all(ol[guard + n:] == -1), "wrote outside the lens"


def test_assemble_errors(capi, dev):
    import torch
    announce("assemble_errors")
    req = to_dev(np.array([1, 3, 5, 7, 9], np.uint64), dev)
    a = (to_dev(np.array([1, 3], np.uint64), dev), torch.ones(2, device=dev), None)
    b = (to_dev(np.array([5, 7, 9], np.uint64), dev), torch.ones(3, device=dev), None)
    out = torch.zeros(5, device=dev)
    assert capi.assemble_pull(req, [b, a], out) == 5
    with pytest.raises(capi.PskvError) as e:  # "lost some servers?" kv_app.h:678
        capi.assemble_pull(req, [a], out)
    assert e.value.code == capi.ESIZE_MISMATCH
    c = (to_dev(np.array([5, 9], np.uint64), dev), torch.ones(2, device=dev), None)
    with pytest.raises(capi.PskvError) as e:  # "unmatched keys size from one server" kv_app.h:672
        capi.assemble_pull(req, [a, c], out)
    assert e.value.code == capi.ESIZE_MISMATCH
