"""Pins the CPU oracle's slicer (oracle/pskv_oracle.cc) WITHOUT a GPU: against the golden
vectors recorded from the reference's own DefaultSlicer, against that function itself when
oracle/_ref is built, against numpy.searchsorted / cumsum, against brute force, and against
the invariants the reference's CHECKs imply."""
import json
import os

import numpy as np
import pytest

from helpers import KMAX, covered_limit, unique_keys

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "slicer_golden.json")
CHECK_TO_STATUS = {542: -1, 549: -2, 551: -2, 249: -2, 533: -6}


def _golden():
    with open(GOLDEN) as f:
        return json.load(f)


@pytest.mark.parametrize("case", _golden()["slicer"], ids=lambda c: c["name"])
def test_golden_vectors(orc, case):
    lens = None if case["lens"] is None else np.array(case["lens"], np.int32)
    rc, pos, vpos, used = orc.slice_status(np.array(case["keys"], np.uint64), np.array(case["range_begin"], np.uint64),
                                           np.array(case["range_end"], np.uint64), lens, case["nvals"])
    if not case["ok"]:
        assert rc == CHECK_TO_STATUS[case["check_line"]], (rc, case["check"])
        return
    assert rc == 0
    assert used.tolist() == case["used"]
    for i, u in enumerate(case["used"]):
        if not u:
            continue  # the reference leaves an unused slice untouched
        assert (int(pos[i]), int(pos[i + 1])) == (case["key_lo"][i], case["key_hi"][i])
        assert (int(vpos[i]), int(vpos[i + 1])) == (case["val_lo"][i], case["val_hi"][i])


@pytest.mark.parametrize("case", _golden()["find_range"], ids=lambda c: "%s_%s" % (c["lower"], c["upper"]))
def test_find_range_golden(orc, case):
    assert orc.find_range(np.array(case["arr"], np.uint64), case["lower"], case["upper"]) == (case["begin"], case["end"])


def test_find_range_doc_example(orc):
    """sarray.h:269-273: FindRange({1,3,5,7,9}, 2, 7) == Range(1,3)."""
    assert orc.find_range(np.array([1, 3, 5, 7, 9], np.uint64), 2, 7) == (1, 3)


def test_server_ranges_closed_form(orc):
    """postoffice.cc:169-180, and the S=4 ranges the reference printed when it was surveyed."""
    b, e = orc.server_ranges(4)
    assert b.tolist() == [0, 4611686018427387903, 9223372036854775806, 13835058055282163709]
    assert e.tolist() == [4611686018427387903, 9223372036854775806, 13835058055282163709, 18446744073709551612]
    for S in (1, 2, 3, 5, 16, 1000):
        b, e = orc.server_ranges(S)
        assert [int(x) for x in b] == [KMAX // S * i for i in range(S)]
        assert [int(x) for x in e] == [KMAX // S * (i + 1) for i in range(S)]
        assert int(e[-1]) == covered_limit(S)


@pytest.mark.parametrize("n,S", [(0, 3), (1, 1), (17, 4), (1000, 16), (100000, 7), (300000, 64)])
def test_against_numpy(orc, n, S):
    """Sorted keys + contiguous ranges: pos = searchsorted(keys, boundaries, 'left'); value offsets are
    pos*k or the prefix sums of lens at pos."""
    rng = np.random.default_rng(n * 31 + S)
    rb, re = orc.server_ranges(S)
    keys = unique_keys(rng, n, S) if n else np.zeros(0, np.uint64)
    bounds = np.concatenate([rb[:1], re])
    want_pos = np.searchsorted(keys, bounds, side="left").astype(np.uint64)
    pos, vpos, used = orc.slice_keys(keys, rb, re, None, 5 * n)
    assert np.array_equal(pos, want_pos) and np.array_equal(vpos, want_pos * np.uint64(5))
    assert np.array_equal(used, (np.diff(want_pos.astype(np.int64)) != 0).astype(np.uint8))
    lens = rng.integers(0, 200, size=n).astype(np.int32)
    csum = np.concatenate([[0], np.cumsum(lens.astype(np.int64))]).astype(np.uint64)
    pos, vpos, used = orc.slice_keys(keys, rb, re, lens, int(lens.sum()))
    assert np.array_equal(pos, want_pos)
    if n:
        assert np.array_equal(vpos, csum[want_pos.astype(np.int64)])
    # invariants of kv_app.h:528-542
    assert pos[0] == 0 and pos[-1] == n and np.all(np.diff(pos.astype(np.int64)) >= 0)
    for i in range(S):
        seg = keys[int(pos[i]):int(pos[i + 1])]
        assert np.all(seg >= rb[i]) and np.all(seg < re[i])


def test_brute_force_small(orc):
    rng = np.random.default_rng(9)
    for _ in range(200):
        S = int(rng.integers(1, 6))
        cuts = np.sort(rng.integers(0, 64, size=S + 1)).astype(np.uint64)
        rb, re = cuts[:-1], cuts[1:]
        keys = np.unique(rng.integers(0, 64, size=int(rng.integers(0, 20)))).astype(np.uint64)
        lens = rng.integers(0, 4, size=keys.size).astype(np.int32)
        nvals = int(lens.sum())
        rc, pos, vpos, used = orc.slice_status(keys, rb, re, lens, nvals)
        covered = [k for k in keys.tolist() if k >= rb[0]]  # keys in front of ranges[0] are skipped (:530)
        if any(k >= re[-1] for k in covered):
            assert rc == -1
            continue
        if keys.size == 0:
            assert rc == 0
            continue
        assert rc == 0
        run = 0  # with lens the value offsets start at 0 whatever was skipped (:546)
        for i in range(S):
            mine = [j for j, k in enumerate(keys.tolist()) if rb[i] <= k < re[i]]
            assert used[i] == (1 if mine else 0)
            assert int(pos[i + 1] - pos[i]) == len(mine)
            if mine:
                assert int(pos[i]) == mine[0]
                assert int(vpos[i]) == run
                run += int(lens[mine].sum())
                assert int(vpos[i + 1]) == run


def test_against_reference_binary(orc):
    """The restatement against the reference's own DefaultSlicer, on random inputs including failing ones."""
    if not orc.have_ref():
        pytest.skip("oracle/_ref is only built where the reference tree is present")
    rng = np.random.default_rng(77)
    for it in range(300):
        S = int(rng.integers(1, 9))
        if it % 3 == 0:
            rb, re = orc.server_ranges(S)
        else:
            cuts = np.sort(rng.integers(0, 1 << 20, size=S + 1)).astype(np.uint64)
            rb, re = cuts[:-1].copy(), cuts[1:].copy()
            if it % 11 == 0 and S > 1:
                rb[1] += np.uint64(1)  # a gap: kv_app.h:533
        hi = min(int(re[-1]) + (50 if it % 5 == 0 else 0), KMAX)
        n = int(rng.integers(0, 60))
        keys = np.unique(rng.integers(0, max(hi, 1), size=n, dtype=np.uint64))
        use_lens = it % 2 == 0
        lens = rng.integers(-1 if it % 13 == 0 else 0, 6, size=keys.size).astype(np.int32) if use_lens else None
        nvals = int(max(lens.sum(), 0)) + int(rng.integers(0, 2)) if use_lens else keys.size * 2 + int(it % 7 == 0)
        if use_lens and it % 17 == 0 and keys.size:
            lens = lens[:-1]
        rc, pos, vpos, used = orc.slice_status(keys, rb, re, lens, nvals)
        ok, klo, khi, vlo, vhi, rused, err = orc.ref_slice(keys, rb, re, lens, nvals)
        assert ok == (rc == 0), (it, rc, err[:200])
        if not ok:
            continue
        assert np.array_equal(used, rused)
        for i in range(S):
            if used[i]:
                assert (pos[i], pos[i + 1], vpos[i], vpos[i + 1]) == (klo[i], khi[i], vlo[i], vhi[i])
