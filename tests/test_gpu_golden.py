"""The committed golden vectors, straight through the C ABI on the GPU.

tests/golden/slicer_golden.json was recorded from the reference's own DefaultSlicer
(kv_app.h:517-572) and tests/golden/store_kat.json holds known answers of the reference's
KVServerDefaultHandle (kv_app.h:440-463). The CPU suite feeds them to the oracle; here they go
to pskv_slice / pskv_push / pskv_pull / pskv_pushpull themselves, host and device buffers."""
import json
import os

import numpy as np
import pytest

from conftest import announce
from helpers import KMAX, from_dev, to_dev

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
CHECK_TO_STATUS = {542: -1, 549: -2, 551: -2, 249: -2, 533: -6}


def _load(name):
    with open(os.path.join(HERE, "golden", name)) as f:
        return json.load(f)


@pytest.mark.parametrize("memkind", ["device", "host"])
@pytest.mark.parametrize("case", _load("slicer_golden.json")["slicer"], ids=lambda c: c["name"])
def test_slicer_golden_vectors(capi, dev, case, memkind):
    announce("slicer_golden", case["name"], memkind)
    keys = np.array(case["keys"], np.uint64)
    lens = None if case["lens"] is None else np.array(case["lens"], np.int32)
    rb, re = np.array(case["range_begin"], np.uint64), np.array(case["range_end"], np.uint64)
    k = to_dev(keys, dev) if memkind == "device" else keys
    l = None if lens is None else (to_dev(lens, dev) if memkind == "device" else lens)
    if not case["ok"]:
        with pytest.raises(capi.PskvError) as e:
            capi.slice_keys(k, rb, re, lens=l, nvals=case["nvals"])
        assert e.value.code == CHECK_TO_STATUS[case["check_line"]], (e.value.code, case["check"])
        return
    pos, vpos, used = capi.slice_keys(k, rb, re, lens=l, nvals=case["nvals"])
    assert used.tolist() == case["used"]
    for i, u in enumerate(case["used"]):
        if not u:
            continue  # the reference leaves an unused slice untouched
        assert (int(pos[i]), int(pos[i + 1])) == (case["key_lo"][i], case["key_hi"][i])
        assert (int(vpos[i]), int(vpos[i + 1])) == (case["val_lo"][i], case["val_hi"][i])


def _run(t, op, memkind, dev):
    """One recorded operation; returns what a pull half answered (numpy) or None."""
    import torch
    keys = np.array(op[1], np.uint64)
    vals = np.array(op[2], np.float32) if len(op) > 2 else None
    if memkind == "host":
        if op[0] == "push":
            t.push(keys, vals)
            return None
        out = np.full(keys.size, np.nan, np.float32)
        if op[0] == "pull":
            t.pull(keys, out)
        else:
            t.pushpull(keys, vals, out)
        return out
    dk = to_dev(keys, dev)
    if op[0] == "push":
        t.push(dk, to_dev(vals, dev))
        t.sync()
        return None
    out = torch.full((keys.size,), float("nan"), dtype=torch.float32, device=dev)
    if op[0] == "pull":
        t.pull(dk, out)
    else:
        t.pushpull(dk, to_dev(vals, dev), out)
    t.sync()
    return from_dev(out)


@pytest.mark.parametrize("memkind", ["device", "host"])
@pytest.mark.parametrize("case", _load("store_kat.json")["cases"], ids=lambda c: c["name"])
def test_store_known_answers(capi, dev, case, memkind):
    announce("store_kat", case["name"], memkind)
    t = capi.Table(capi.MODE_SCALAR, initial_capacity=16)
    if "ops" in case:
        out = None
        for op in case["ops"]:
            got = _run(t, op, memkind, dev)
            out = got if got is not None else out
        if "expect_bits" in case:
            assert ["%08x" % b for b in out.view(np.uint32)] == case["expect_bits"], case["name"]
        else:
            assert out.tolist() == case["expect"], case["name"]
        assert t.size()[0] == case["expect_size"], case["name"]
        return
    # tests/test_kv_app.cc:27-60 with the values of the plumbing run
    n = case["n"]
    keys = np.uint64(KMAX // n) * np.arange(n, dtype=np.uint64)
    vals = np.full(n, case["val"], np.float32)
    for _ in range(case["repeat_push"]):
        _run(t, ["push", keys, vals], memkind, dev)
    out = _run(t, ["pull", keys], memkind, dev)
    assert np.all(out == np.float32(case["expect_all"]))
    for _ in range(case["then_pushpull"]):
        out = _run(t, ["pushpull", keys, vals], memkind, dev)
    assert np.all(out == np.float32(case["expect_all_after"]))
    assert t.size()[0] == n
