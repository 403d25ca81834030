"""Pins the CPU oracle's ordered match (ParallelOrderedMatch, include/ps/internal/parallel_kv_match.h:29-120)
WITHOUT a GPU. The reference's header does not compile (assign_op.h:27-41 names undeclared variables), so there
is no build of it to compare with; the oracle is pinned by what the documented contract fixes
(`if (dst_key[i] == src_key[j]) dst_val[i] op= src_val[j]`, :82-86): a numpy searchsorted model, closed forms,
and a brute-force double loop on small inputs."""
import numpy as np
import pytest

from helpers import assert_bits_equal, unique_keys

OPS = {0: lambda d, s: s, 1: lambda d, s: d + s, 2: lambda d, s: d - s, 3: lambda d, s: d * s,
       4: lambda d, s: d / s}


def numpy_model(sk, sv, dk, dv, k, op):
    out = dv.reshape(-1, k).copy()
    src = sv.reshape(-1, k)
    if sk.size and dk.size:
        j = np.searchsorted(sk, dk)
        hit = (j < sk.size) & (sk[np.minimum(j, sk.size - 1)] == dk)
        with np.errstate(all="ignore"):
            out[hit] = OPS[op](out[hit], src[j[hit]]).astype(np.float32)
        return out.reshape(-1), int(hit.sum()) * k
    return out.reshape(-1), 0


def key_sets(rng, n_src, n_dst, shared):
    pool = unique_keys(rng, n_src + n_dst)
    both = rng.choice(pool, size=min(shared, n_src, n_dst), replace=False)
    rest = np.setdiff1d(pool, both)
    rng.shuffle(rest)
    sk = np.sort(np.concatenate([both, rest[:n_src - both.size]]))
    dk = np.sort(np.concatenate([both, rest[n_src - both.size:n_src - both.size + n_dst - both.size]]))
    return sk, dk


@pytest.mark.parametrize("op", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("k", [1, 2, 7])
def test_against_the_numpy_model(orc, op, k):
    rng = np.random.default_rng(100 * op + k)
    for n_src, n_dst, shared in [(0, 5, 0), (5, 0, 0), (1, 1, 1), (1, 1, 0), (300, 200, 120), (200, 3000, 200),
                                 (3000, 200, 150), (1000, 1000, 0), (777, 777, 777)]:
        sk, dk = key_sets(rng, n_src, n_dst, shared)
        sv = rng.standard_normal(sk.size * k).astype(np.float32)
        dv = rng.standard_normal(dk.size * k).astype(np.float32)
        rc, got, matched = orc.ordered_match(sk, sv, dk, dv, k, op)
        want, want_n = numpy_model(sk, sv, dk, dv, k, op)
        assert rc == 0 and matched == want_n, (n_src, n_dst, shared)
        assert_bits_equal(got, want, "n_src %d n_dst %d shared %d" % (n_src, n_dst, shared))


def test_closed_forms(orc):
    """Equal key sets: every value is touched and `matched` counts VALUES (k per key, :52).
    Disjoint key sets: nothing moves. ASSIGN of a subset leaves the other destination values."""
    keys = np.array([1, 3, 5, 7, 9], np.uint64)
    sv = np.arange(10, dtype=np.float32) + 1
    dv = np.full(10, 100.0, np.float32)
    rc, got, n = orc.ordered_match(keys, sv, keys, dv, 2, orc.OP_PLUS)
    assert rc == 0 and n == 10 and got.tolist() == (100 + sv).tolist()
    rc, got, n = orc.ordered_match(keys, sv, keys + np.uint64(1), dv, 2, orc.OP_ASSIGN)
    assert rc == 0 and n == 0 and got.tolist() == dv.tolist()
    rc, got, n = orc.ordered_match(np.array([3, 9, 11], np.uint64), np.array([30, 90, 110], np.float32),
                                   keys, np.zeros(5, np.float32), 1, orc.OP_ASSIGN)
    assert rc == 0 and n == 2 and got.tolist() == [0, 30, 0, 0, 90]
    # the largest key and key 0 are keys like any other
    ends = np.array([0, 2**64 - 1], np.uint64)
    rc, got, n = orc.ordered_match(ends, np.array([4, 8], np.float32), ends, np.array([1, 2], np.float32), 1,
                                   orc.OP_TIMES)
    assert rc == 0 and n == 2 and got.tolist() == [4, 16]
    # the bit operators of assign_op.h:20-22 are for integers only (:38)
    assert orc.ordered_match(keys, sv[:5], keys, dv[:5], 1, 5)[0] != 0


def test_against_a_double_loop(orc):
    rng = np.random.default_rng(7)
    for _ in range(30):
        sk = np.unique(rng.integers(0, 60, size=int(rng.integers(0, 30))).astype(np.uint64))
        dk = np.unique(rng.integers(0, 60, size=int(rng.integers(0, 30))).astype(np.uint64))
        k = int(rng.integers(1, 4))
        sv = rng.integers(1, 9, size=sk.size * k).astype(np.float32)
        dv = rng.integers(1, 9, size=dk.size * k).astype(np.float32)
        want = dv.copy()
        count = 0
        for i in range(dk.size):
            for j in range(sk.size):
                if dk[i] == sk[j]:
                    want[i * k:(i + 1) * k] -= sv[j * k:(j + 1) * k]
                    count += k
        rc, got, n = orc.ordered_match(sk, sv, dk, dv, k, orc.OP_MINUS)
        assert rc == 0 and n == count
        assert_bits_equal(got, want, "double loop")
