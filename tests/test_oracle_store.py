"""Pins the CPU oracle's request handle WITHOUT a GPU: a dict of numpy float32 as the model of
std::unordered_map<Key,float>, the closed forms of the reference's own test, recorded
known answers, and for the multi-float stores reduction to the scalar case and numpy sums."""
import json
import os

import numpy as np
import pytest

from helpers import KMAX, assert_bits_equal, unique_keys

KAT = os.path.join(os.path.dirname(__file__), "golden", "store_kat.json")


class DictModel:
    """store[key] += v / out = store[key] with float32 arithmetic (kv_app.h:451-459)."""

    def __init__(self):
        self.d = {}

    def handle(self, push, pull, keys, vals=None):
        out = []
        for i, k in enumerate(keys.tolist()):
            if push:
                self.d[k] = np.float32(self.d.get(k, np.float32(0.0)) + np.float32(vals[i]))
            if pull:
                self.d.setdefault(k, np.float32(0.0))
                out.append(self.d[k])
        return np.array(out, np.float32)


def test_scalar_against_dict_model(orc):
    rng = np.random.default_rng(1)
    o = orc.Store(orc.MODE_SCALAR)
    m = DictModel()
    universe = unique_keys(rng, 3000)
    for it in range(40):
        keys = np.sort(rng.choice(universe, size=int(rng.integers(0, 700)), replace=False))
        vals = rng.standard_normal(keys.size).astype(np.float32)
        push, pull = [(True, False), (False, True), (True, True)][it % 3]
        rc, out, _, got = o.handle(push, pull, keys, vals if push else None)
        want = m.handle(push, pull, keys, vals)
        assert rc == 0
        if pull:
            assert got == keys.size
            assert_bits_equal(out, want, "op %d" % it)
    dk, dl, dv = o.dump()
    assert dk.tolist() == sorted(m.d)
    assert_bits_equal(dv, np.array([m.d[k] for k in sorted(m.d)], np.float32), "dump")
    assert o.size() == (len(m.d), len(m.d))


def test_scalar_request_that_repeats_keys(orc):
    """The reference's handle is a loop over the request (kv_app.h:451-459), so a request that
    repeats a key has a defined result: every occurrence adds, and with push+pull each position
    shows the sum so far. Answer worked out by hand, then the dict model on random runs."""
    o = orc.Store(orc.MODE_SCALAR)
    keys = np.array([5, 9, 9, 9, 12, 12, 40], np.uint64)
    rc, out, _, _ = o.handle(True, True, keys, np.ones(7, np.float32), out_cap=7)
    assert rc == 0 and out.tolist() == [1, 1, 2, 3, 1, 2, 1]
    rc, out, _, _ = o.handle(False, True, keys, out_cap=7)
    assert rc == 0 and out.tolist() == [1, 3, 3, 3, 2, 2, 1]
    rng = np.random.default_rng(2)
    m = DictModel()
    o = orc.Store(orc.MODE_SCALAR)
    universe = unique_keys(rng, 200)
    for it in range(30):
        keys = np.sort(universe[rng.integers(0, universe.size, size=int(rng.integers(1, 900)))])
        vals = rng.standard_normal(keys.size).astype(np.float32)
        push, pull = [(True, False), (False, True), (True, True)][it % 3]
        rc, out, _, _ = o.handle(push, pull, keys, vals if push else None, out_cap=keys.size)
        want = m.handle(push, pull, keys, vals)
        assert rc == 0
        if pull:
            assert_bits_equal(out, want, "op %d" % it)
    assert_bits_equal(o.dump()[2], np.array([m.d[k] for k in sorted(m.d)], np.float32), "dump")


def test_recorded_known_answers(orc):
    with open(KAT) as f:
        kat = json.load(f)
    for case in kat["cases"]:
        o = orc.Store(orc.MODE_SCALAR)
        if "ops" in case:
            out = None
            for op in case["ops"]:
                keys = np.array(op[1], np.uint64)
                if op[0] == "push":
                    o.push(keys, np.array(op[2], np.float32))
                elif op[0] == "pull":
                    out, _ = o.pull(keys)
                else:
                    out, _ = o.pushpull(keys, np.array(op[2], np.float32))
            if "expect_bits" in case:
                assert ["%08x" % b for b in out.view(np.uint32)] == case["expect_bits"], case["name"]
            else:
                assert out.tolist() == case["expect"], case["name"]
            assert o.size()[0] == case["expect_size"], case["name"]
        else:  # tests/test_kv_app.cc:27-60
            n = case["n"]
            keys = np.uint64(KMAX // n) * np.arange(n, dtype=np.uint64)
            vals = np.full(n, case["val"], np.float32)
            for _ in range(case["repeat_push"]):
                o.push(keys, vals)
            out, _ = o.pull(keys)
            assert np.all(out == np.float32(case["expect_all"]))
            for _ in range(case["then_pushpull"]):
                out, _ = o.pushpull(keys, vals)
            assert np.all(out == np.float32(case["expect_all_after"]))


def test_reference_test_closed_form(orc):
    """tests/test_kv_app.cc: 10,000 keys kMaxKey/num*i + rank, vals rand()%1000; 50 pushes -> 50*v,
    50 push+pulls more -> 100*v, exactly (small integers add without rounding)."""
    num = 10000
    keys = np.uint64(KMAX // num) * np.arange(num, dtype=np.uint64)
    vals = np.random.default_rng(7).integers(0, 1000, size=num).astype(np.float32)
    o = orc.Store(orc.MODE_SCALAR)
    for _ in range(50):
        o.push(keys, vals)
    assert np.array_equal(o.pull(keys)[0], vals * 50)
    for _ in range(50):
        out, _ = o.pushpull(keys, vals)
    assert np.array_equal(out, vals * 100)


def test_scalar_size_check(orc):
    o = orc.Store(orc.MODE_SCALAR)
    assert o.handle(True, False, np.array([1, 2], np.uint64), np.ones(3, np.float32))[0] == orc.ESIZE_MISMATCH  # :447
    assert o.size() == (0, 0)
    rc, _, _, need = o.handle(False, True, np.array([1, 2], np.uint64), out_cap=1)
    assert rc == orc.ESIZE_MISMATCH and need == 2 and o.size() == (2, 2)


def test_fixed_k1_equals_scalar(orc):
    rng = np.random.default_rng(3)
    a, b = orc.Store(orc.MODE_SCALAR), orc.Store(orc.MODE_FIXED)
    universe = unique_keys(rng, 500)
    for it in range(12):
        keys = np.sort(rng.choice(universe, size=200, replace=False))
        vals = rng.standard_normal(200).astype(np.float32)
        if it % 4 == 3:
            assert_bits_equal(a.pull(keys)[0], b.pull(keys)[0], "pull")
        else:
            a.push(keys, vals)
            b.push(keys, vals)
    assert np.array_equal(a.dump()[0], b.dump()[0])
    assert_bits_equal(a.dump()[2], b.dump()[2], "dump")


@pytest.mark.parametrize("k", [2, 7, 64])
def test_fixed_against_numpy(orc, k):
    """Row r of key i is vals[i*k:(i+1)*k] (kv_app.h:17-22); sums are sequential float32 adds from a
    zero row; a pull of an absent key creates a zero row."""
    rng = np.random.default_rng(k)
    universe = unique_keys(rng, 300)
    o = orc.Store(orc.MODE_FIXED)
    model = {}
    for it in range(8):
        keys = np.sort(rng.choice(universe, size=120, replace=False))
        vals = rng.uniform(-1, 1, size=120 * k).astype(np.float32)
        o.push(keys, vals)
        for i, key in enumerate(keys.tolist()):
            model[key] = (model.get(key, np.zeros(k, np.float32)) + vals[i * k:(i + 1) * k]).astype(np.float32)
    keys = np.sort(rng.choice(universe, size=150, replace=False))
    out, _ = o.pull(keys)
    want = np.concatenate([model.setdefault(key, np.zeros(k, np.float32)) for key in keys.tolist()])
    assert_bits_equal(out, want, "fixed")
    assert o.size() == (len(model), len(model) * k)
    assert o.handle(True, False, keys, np.zeros(150 * k + 1, np.float32))[0] == orc.ESIZE_MISMATCH  # :549
    assert o.handle(True, False, keys, np.zeros(150 * (k + 1), np.float32))[0] == orc.ESIZE_MISMATCH


def test_fixed_doc_example(orc):
    """kv_app.h:89-96: {1:(1.1,1.2), 3:(3.1,3.2)}."""
    o = orc.Store(orc.MODE_FIXED)
    o.push(np.array([1, 3], np.uint64), np.array([1.1, 1.2, 3.1, 3.2], np.float32))
    out, _ = o.pull(np.array([3, 1], np.uint64)[::-1].copy())
    assert_bits_equal(out, np.array([1.1, 1.2, 3.1, 3.2], np.float32) + np.float32(0), "doc")


def test_varlen_against_numpy(orc):
    """Row of key i starts at sum(lens[:i]) (kv_app.h:24-31). Absent keys answer length 0 and are
    not created; a changed length is refused and changes no value."""
    rng = np.random.default_rng(5)
    universe = unique_keys(rng, 400)
    len_of = {k: int(l) for k, l in zip(universe.tolist(), rng.integers(0, 40, size=universe.size))}
    o = orc.Store(orc.MODE_VARLEN)
    model = {}
    for it in range(6):
        keys = np.sort(rng.choice(universe, size=150, replace=False))
        lens = np.array([len_of[k] for k in keys.tolist()], np.int32)
        vals = rng.normal(0, 0.1, size=int(lens.sum())).astype(np.float32)
        o.push(keys, vals, lens)
        off = 0
        for key, l in zip(keys.tolist(), lens.tolist()):
            model[key] = (model.get(key, np.zeros(l, np.float32)) + vals[off:off + l]).astype(np.float32)
            off += l
    keys = np.sort(rng.choice(universe, size=300, replace=False))
    out, out_lens = o.pull(keys)
    want_lens = [len(model[k]) if k in model else 0 for k in keys.tolist()]
    assert out_lens.tolist() == want_lens
    want = np.concatenate([model[k] for k in keys.tolist() if k in model] + [np.zeros(0, np.float32)])
    assert_bits_equal(out, want, "varlen")
    assert o.size()[0] == len(model)
    # refused push: one present key with a different length, one absent key
    present = next(k for k in keys.tolist() if k in model)
    absent = next(k for k in sorted(universe.tolist()) if k not in model)
    req = np.array(sorted([present, absent]), np.uint64)
    lens = np.array([len(model[present]) + 1 if k == present else 3 for k in req.tolist()], np.int32)
    before = o.pull(np.array([present], np.uint64))[0].copy()
    assert o.handle(True, False, req, np.ones(int(lens.sum()), np.float32), lens)[0] == orc.ELEN_CHANGED
    assert_bits_equal(o.pull(np.array([present], np.uint64))[0], before, "unchanged")
    out, out_lens = o.pull(np.array([absent], np.uint64))
    assert out_lens.tolist() == [3] and out.tolist() == [0.0, 0.0, 0.0]
    # size checks
    assert o.handle(True, False, req, np.ones(5, np.float32), lens[:1])[0] == orc.ESIZE_MISMATCH
    assert o.handle(True, False, req, np.ones(2, np.float32), np.array([1, 2], np.int32))[0] == orc.ESIZE_MISMATCH
    assert o.handle(True, False, req, np.ones(2, np.float32), np.array([3, -1], np.int32))[0] == orc.EINVAL


def test_assemble_pull_against_numpy(orc):
    """kv_app.h:663-714: responses in any order are ordered by first key and concatenated."""
    rng = np.random.default_rng(8)
    keys = unique_keys(rng, 1000)
    lens = rng.integers(0, 6, size=1000).astype(np.int32)
    vals = rng.standard_normal(int(lens.sum())).astype(np.float32)
    cuts = [0, 100, 101, 640, 1000]
    off = np.concatenate([[0], np.cumsum(lens)])
    parts = [(keys[a:b], vals[off[a]:off[b]], lens[a:b]) for a, b in zip(cuts[:-1], cuts[1:])]
    order = [2, 0, 3, 1]
    rc, out, out_lens = orc.assemble_pull(keys, [parts[i] for i in order], True)
    assert rc == 0 and np.array_equal(out_lens, lens)
    assert_bits_equal(out, vals, "assembled")
    assert orc.assemble_pull(keys, [parts[0], parts[1], parts[3]], True)[0] == orc.ESIZE_MISMATCH  # :678
    bad = (keys[100:640:2], vals[:1], lens[:1])
    assert orc.assemble_pull(keys, [parts[0], bad], False)[0] == orc.ESIZE_MISMATCH  # :672
