"""Shared helpers of the parity tests: seeded generators and bit-level comparison."""
import numpy as np

KMAX = (1 << 64) - 1


def covered_limit(S):
    """Keys at or above this are not covered by the S stock ranges (postoffice.cc:169-180)."""
    return (KMAX // S) * S


def unique_keys(rng, n, S=1, lo=0):
    """n sorted unique uint64 keys uniform over the covered key space."""
    hi = covered_limit(S)
    keys = np.unique(rng.integers(lo, hi, size=int(n * 1.01) + 16, dtype=np.uint64))
    while keys.size < n:
        more = rng.integers(lo, hi, size=n, dtype=np.uint64)
        keys = np.unique(np.concatenate([keys, more]))
    if keys.size > n:
        keys = np.sort(rng.choice(keys, size=n, replace=False))
    return keys


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def assert_bits_equal(got, want, what=""):
    got = np.ascontiguousarray(got, dtype=np.float32)
    want = np.ascontiguousarray(want, dtype=np.float32)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    bad = np.flatnonzero(bits(got) != bits(want))
    assert bad.size == 0, "%s: %d of %d floats differ, first at %d: got %r want %r" % (
        what, bad.size, got.size, bad[0], got[bad[0]], want[bad[0]])


def to_dev(a, dev):
    import torch
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint64:
        a = a.view(np.int64)
    return torch.from_numpy(a).to(dev)


def from_dev(t):
    a = t.cpu().numpy()
    return a
