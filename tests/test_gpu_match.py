"""pskv_match (the ordered match of parallel_kv_match.h:29-120 on the GPU) against the CPU oracle, bit for bit,
through the C ABI: every operator, k = 1 and longer values (vector and scalar row paths), key sets of every
relative density (source stretch staged in LDS or searched in place), both memory kinds, and at the size of a
model through properties that do not depend on it."""
import numpy as np
import pytest

from conftest import announce
from helpers import assert_bits_equal, from_dev, to_dev, unique_keys
from test_oracle_match import key_sets, numpy_model

pytestmark = pytest.mark.gpu

SHAPES = [(1, 1, 1), (1, 1, 0), (300, 200, 120), (200, 30000, 200), (60000, 900, 700), (5000, 5000, 0),
          (4097, 4097, 4097), (100000, 100000, 50000)]


def values(rng, n, op):
    v = rng.standard_normal(n).astype(np.float32)
    if op == 4:  # keep divisors away from zero: the bits of a NaN from 0/0 differ between CPU and GPU
        v = np.where(np.abs(v) < 0.01, np.float32(0.5), v).astype(np.float32)
    return v


def run(capi, dev, memkind, sk, sv, dk, dv, k, op, shift=0):
    if memkind == "host":
        got = dv.copy()
        n = capi.match(sk, sv, dk, got, k, op)
        return got, n
    import torch
    room = torch.zeros(dv.size + 8, dtype=torch.float32, device=dev)
    d = room[shift:shift + dv.size]
    d.copy_(to_dev(dv, dev))
    n = capi.match(to_dev(sk, dev), to_dev(sv, dev), to_dev(dk, dev), d, k, op)
    return from_dev(d), n


@pytest.mark.parametrize("memkind", ["device", "host"])
@pytest.mark.parametrize("op", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("k", [1, 4, 7, 64])
def test_match_against_the_oracle(capi, orc, dev, memkind, op, k):
    announce("match", memkind, op, k)
    rng = np.random.default_rng(1000 * op + k)
    for n_src, n_dst, shared in SHAPES:
        if k == 64 and max(n_src, n_dst) > 30000:
            continue
        sk, dk = key_sets(rng, n_src, n_dst, shared)
        sv, dv = values(rng, sk.size * k, op), values(rng, dk.size * k, op)
        rc, want, want_n = orc.ordered_match(sk, sv, dk, dv, k, op)
        assert rc == 0
        got, n = run(capi, dev, memkind, sk, sv, dk, dv, k, op)
        assert n == want_n, (n_src, n_dst, shared)
        assert_bits_equal(got, want, "n_src %d n_dst %d shared %d" % (n_src, n_dst, shared))


def test_match_edges(capi, orc, dev):
    """Empty sides, the keys 0 and 2^64-1, a destination buffer that is not 16-byte aligned (k = 4 then
    takes the scalar row path), and what the host refuses."""
    announce("match_edges")
    keys = np.array([0, 5, 2**64 - 1], np.uint64)
    sv = np.array([1, 2, 3], np.float32)
    dv = np.array([10, 20, 30], np.float32)
    got, n = run(capi, dev, "device", keys, sv, keys, dv, 1, capi.OP_MINUS)
    assert n == 3 and got.tolist() == [9, 18, 27]
    empty_k, empty_v = np.zeros(0, np.uint64), np.zeros(0, np.float32)
    assert capi.match(empty_k, empty_v, keys, dv.copy(), 1, capi.OP_ASSIGN) == 0
    assert capi.match(keys, sv, empty_k, empty_v.copy(), 1, capi.OP_ASSIGN) == 0
    rng = np.random.default_rng(5)
    sk, dk = key_sets(rng, 3000, 2000, 1500)
    sv4, dv4 = values(rng, sk.size * 4, 1), values(rng, dk.size * 4, 1)
    _, want, want_n = orc.ordered_match(sk, sv4, dk, dv4, 4, orc.OP_PLUS)
    got, n = run(capi, dev, "device", sk, sv4, dk, dv4, 4, capi.OP_PLUS, shift=1)
    assert n == want_n
    assert_bits_equal(got, want, "unaligned destination")
    with pytest.raises(capi.PskvError) as e:
        capi.match(keys, sv, keys, dv.copy(), 1, 5)  # AND: integers only (assign_op.h:38)
    assert e.value.code == capi.EINVAL
    with pytest.raises(capi.PskvError):
        capi.match(keys, np.zeros(0, np.float32), keys, np.zeros(0, np.float32), 0, 0)


def test_match_at_the_size_of_a_model(capi, dev):
    """16M destination keys against 12M source keys (8M shared), k = 1 and k = 8, on the device. Checked
    against numpy's searchsorted, and through properties: matching a key set with itself touches every value,
    MINUS after PLUS of integer-valued floats restores the destination, ASSIGN is idempotent."""
    import torch
    announce("match_large")
    rng = np.random.default_rng(11)
    pool = unique_keys(rng, 20_000_000)
    perm = rng.permutation(pool.size)
    sk = np.sort(pool[perm[:12_000_000]])
    dk = np.sort(pool[perm[4_000_000:20_000_000]])
    for k in (1, 8):
        sv = rng.integers(-50, 50, size=sk.size * k).astype(np.float32)
        dv = rng.integers(-50, 50, size=dk.size * k).astype(np.float32)
        want, want_n = numpy_model(sk, sv, dk, dv, k, 1)
        d_sk, d_sv, d_dk, d_dv = to_dev(sk, dev), to_dev(sv, dev), to_dev(dk, dev), to_dev(dv, dev)
        n = capi.match(d_sk, d_sv, d_dk, d_dv, k, capi.OP_PLUS)
        assert n == want_n == 8_000_000 * k
        assert_bits_equal(from_dev(d_dv), want, "plus, k=%d" % k)
        assert capi.match(d_sk, d_sv, d_dk, d_dv, k, capi.OP_MINUS) == want_n
        assert_bits_equal(from_dev(d_dv), dv, "minus after plus restores, k=%d" % k)
        assert capi.match(d_sk, d_sv, d_dk, d_dv, k, capi.OP_ASSIGN) == want_n
        once = from_dev(d_dv)
        assert capi.match(d_sk, d_sv, d_dk, d_dv, k, capi.OP_ASSIGN) == want_n
        assert_bits_equal(from_dev(d_dv), once, "assign twice, k=%d" % k)
        d_self = torch.ones(dk.size * k, dtype=torch.float32, device=dev)
        assert capi.match(d_dk, d_dv, d_dk, d_self, k, capi.OP_TIMES) == dk.size * k
        assert_bits_equal(from_dev(d_self), once, "a key set against itself, k=%d" % k)
