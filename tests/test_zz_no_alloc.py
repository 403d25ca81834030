"""The slicer entry point that allocates nothing (pskv_slice_noalloc) against pskv_slice,
through the C ABI: identical positions, value offsets, `first` flags and status codes. Every
case makes two calls in a row on the same GPU, the second with a smaller input, because all
calls share one fixed working array inside the library."""
import json
import os

import numpy as np
import pytest

from conftest import announce
from helpers import to_dev, unique_keys

pytestmark = pytest.mark.gpu

CHECK_TO_STATUS = {542: -1, 549: -2, 551: -2, 249: -2, 533: -6}


def _load(name):
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", name)) as f:
        return json.load(f)


def _reference(capi, dk, rb, re, dl, nvals):
    """(status, pos, val_pos, used) of the allocating entry point."""
    try:
        pos, vpos, used = capi.slice_keys(dk, rb, re, lens=dl, nvals=nvals)
    except capi.PskvError as e:
        return e.code, None, None, None
    return 0, pos, vpos, used


def _noalloc(capi, dev, dk, rb, re, dl, nvals, stream=None):
    import torch
    S = len(rb)
    # outputs start as garbage so that every word the call leaves untouched shows
    pos = torch.full((S + 1,), -7, dtype=torch.int64, device=dev)
    vpos = torch.full((S + 1,), -7, dtype=torch.int64, device=dev)
    used = torch.full((S,), 9, dtype=torch.uint8, device=dev)
    status = torch.full((1,), 12345, dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    capi.slice_keys_noalloc(dk, rb, re, pos, vpos, used, status, lens=dl, nvals=nvals, stream=stream)
    torch.cuda.synchronize()
    return (int(status.item()), pos.cpu().numpy().view(np.uint64), vpos.cpu().numpy().view(np.uint64),
            used.cpu().numpy())


def _check_pair(capi, dev, keys, lens, nvals, S, stream=None):
    rb, re = capi.server_ranges(S)
    dk = to_dev(keys, dev)
    dl = None if lens is None else to_dev(lens, dev)
    want = _reference(capi, dk, rb, re, dl, nvals)
    got = _noalloc(capi, dev, dk, rb, re, dl, nvals, stream)
    assert got[0] == want[0], (got[0], want[0])
    if want[0] == 0:
        assert np.array_equal(got[1], want[1]), (got[1], want[1])
        assert np.array_equal(got[2], want[2]), (got[2], want[2])
        assert np.array_equal(got[3], want[3])
    elif want[0] == capi.EUNCOVERED_KEY:
        # positions and flags are defined even then; compare them with numpy
        p = np.concatenate([[np.searchsorted(keys, rb[0])], np.searchsorted(keys, re)])
        assert np.array_equal(got[1].astype(np.int64), p.astype(np.int64))
        assert np.array_equal(got[3].astype(bool), np.diff(p) > 0)


@pytest.mark.parametrize("n1,S1,n2,S2", [(200000, 16, 5000, 4), (1000003, 4, 77, 1), (300000, 100, 1000, 31),
                                         (50000, 1024, 50000, 33), (4096, 32, 0, 3)])
def test_no_alloc_matches_slice_twice_in_a_row(capi, dev, n1, S1, n2, S2):
    announce("no_alloc_pair", n1, S1, n2, S2)
    rng = np.random.default_rng(n1 + S1)
    for n, S in ((n1, S1), (n2, S2)):
        keys = unique_keys(rng, n, S) if n else np.zeros(0, np.uint64)
        lens = rng.choice(np.array([0, 8, 16, 32, 64, 128], np.int32), size=n).astype(np.int32)
        _check_pair(capi, dev, keys, lens, int(lens.sum()), S)  # lens
        _check_pair(capi, dev, keys, None, 3 * n, S)            # fixed k = 3
        _check_pair(capi, dev, keys, None, 0, S)                # a pull request: no values


def test_no_alloc_status_codes(capi, dev):
    """The data-dependent failures arrive in *status with pskv_slice's codes; what the host can
    decide alone comes back from the call itself."""
    import torch
    announce("no_alloc_status")
    rng = np.random.default_rng(5)
    S = 8
    rb, re = capi.server_ranges(S)
    keys = unique_keys(rng, 10000, S)
    lens = rng.integers(0, 9, size=keys.size).astype(np.int32)
    total = int(lens.sum())
    # a key beyond the last range (kv_app.h:542), then a good call: the status is rewritten
    bad = np.concatenate([keys, np.array([(1 << 64) - 2], np.uint64)])
    _check_pair(capi, dev, bad, None, 2 * bad.size, S)
    _check_pair(capi, dev, keys, lens, total, S)
    # values that do not divide over the keys (kv_app.h:549), lens of another size (:551), lens
    # that reach past the values (sarray.h:249), negative lens
    _check_pair(capi, dev, keys, None, 2 * keys.size + 1, S)
    _check_pair(capi, dev, keys, lens[:-1], total, S)
    _check_pair(capi, dev, keys, lens, total - 1, S)
    neg = lens.copy()
    neg[::7] = -3
    _check_pair(capi, dev, keys, neg, total, S)
    _check_pair(capi, dev, keys[:100], lens[:100], int(lens[:100].sum()), S)
    # uncovered AND indivisible: the coverage check comes first, as in the reference
    _check_pair(capi, dev, bad, None, 2 * bad.size + 1, S)
    # host-side refusals
    dk = to_dev(keys, dev)
    out = [torch.zeros(2000, dtype=torch.int64, device=dev), torch.zeros(2000, dtype=torch.int64, device=dev),
           torch.zeros(2000, dtype=torch.uint8, device=dev), torch.zeros(1, dtype=torch.int32, device=dev)]
    rb2, re2 = capi.server_ranges(capi.SLICE_NOALLOC_MAX_RANGES + 1)
    with pytest.raises(capi.PskvError) as e:
        capi.slice_keys_noalloc(dk, rb2, re2, *out)
    assert e.value.code == capi.EINVAL and "at most" in str(e.value)
    gap_b, gap_e = rb.copy(), re.copy()
    gap_e[2] -= np.uint64(1)
    with pytest.raises(capi.PskvError) as e:
        capi.slice_keys_noalloc(dk, gap_b, gap_e, *out)
    assert e.value.code == capi.ERANGE_GAP
    with pytest.raises(capi.PskvError) as e:
        capi.slice_keys_noalloc(dk, rb[:0], re[:0], *out)
    assert e.value.code == capi.EINVAL


def test_no_alloc_on_a_caller_stream(capi, dev):
    """Enqueued on the caller's stream, nothing waits inside the call: two calls queued back to
    back on one stream each leave their own answer."""
    import torch
    announce("no_alloc_stream")
    rng = np.random.default_rng(11)
    s = torch.cuda.Stream()
    res = []
    for n, S in ((400000, 64), (3000, 5)):
        keys = unique_keys(rng, n, S)
        lens = rng.integers(0, 5, size=n).astype(np.int32)
        _check_pair(capi, dev, keys, lens, int(lens.sum()), S, stream=s.cuda_stream)
    # queued without a wait in between
    sets = []
    for n, S in ((400000, 64), (3000, 5)):
        keys = unique_keys(rng, n, S)
        lens = rng.integers(0, 5, size=n).astype(np.int32)
        rb, re = capi.server_ranges(S)
        dk, dl = to_dev(keys, dev), to_dev(lens, dev)
        o = (torch.zeros(S + 1, dtype=torch.int64, device=dev), torch.zeros(S + 1, dtype=torch.int64, device=dev),
             torch.zeros(S, dtype=torch.uint8, device=dev), torch.full((1,), 7, dtype=torch.int32, device=dev))
        sets.append((keys, lens, rb, re, dk, dl, o))
    torch.cuda.synchronize()
    for keys, lens, rb, re, dk, dl, o in sets:
        capi.slice_keys_noalloc(dk, rb, re, *o, lens=dl, nvals=int(lens.sum()), stream=s.cuda_stream)
    s.synchronize()
    for keys, lens, rb, re, dk, dl, o in sets:
        want = _reference(capi, dk, rb, re, dl, int(lens.sum()))
        assert int(o[3].item()) == 0 and want[0] == 0
        assert np.array_equal(o[0].cpu().numpy().view(np.uint64), want[1])
        assert np.array_equal(o[1].cpu().numpy().view(np.uint64), want[2])
        assert np.array_equal(o[2].cpu().numpy(), want[3])


@pytest.mark.parametrize("case", _load("slicer_golden.json")["slicer"], ids=lambda c: c["name"])
def test_slicer_golden_vectors_no_alloc(capi, dev, case):
    """The vectors recorded from the reference's own DefaultSlicer (kv_app.h:517-572) through the
    entry point that allocates nothing."""
    import torch
    announce("slicer_golden_no_alloc", case["name"])
    keys = np.array(case["keys"], np.uint64)
    lens = None if case["lens"] is None else np.array(case["lens"], np.int32)
    rb, re = np.array(case["range_begin"], np.uint64), np.array(case["range_end"], np.uint64)
    S = rb.size
    pos = torch.full((S + 1,), -1, dtype=torch.int64, device=dev)
    vpos = torch.full((S + 1,), -1, dtype=torch.int64, device=dev)
    used = torch.full((S,), 7, dtype=torch.uint8, device=dev)
    status = torch.full((1,), 99, dtype=torch.int32, device=dev)
    dk = to_dev(keys, dev)
    dl = None if lens is None else to_dev(lens, dev)
    torch.cuda.synchronize()
    try:
        capi.slice_keys_noalloc(dk, rb, re, pos, vpos, used, status, lens=dl, nvals=case["nvals"])
        torch.cuda.synchronize()
        rc = int(status.item())
    except capi.PskvError as e:  # what the host alone can decide (a gap between ranges)
        rc = e.code
    if not case["ok"]:
        assert rc == CHECK_TO_STATUS[case["check_line"]], (rc, case["check"])
        return
    assert rc == 0
    pos, vpos = pos.cpu().numpy(), vpos.cpu().numpy()
    assert used.cpu().numpy().tolist() == case["used"]
    for i, u in enumerate(case["used"]):
        if not u:
            continue
        assert (int(pos[i]), int(pos[i + 1])) == (case["key_lo"][i], case["key_hi"][i])
        assert (int(vpos[i]), int(vpos[i + 1])) == (case["val_lo"][i], case["val_hi"][i])
