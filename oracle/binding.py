"""ctypes binding of the CPU oracle. TEST INFRASTRUCTURE ONLY: imported by tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg, never by the product."""
import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "liboracle.so")
REF_LIB = os.path.join(HERE, "_ref", "libpskv_ref.so")

OK, EUNCOVERED_KEY, ESIZE_MISMATCH, ENOMEM, EINVAL, ERANGE_GAP, ELEN_CHANGED = 0, -1, -2, -3, -5, -6, -7
MODE_SCALAR, MODE_FIXED, MODE_VARLEN = 0, 1, 2

_lib = None
_ref = None


class OracleError(RuntimeError):
    def __init__(self, code):
        super().__init__("oracle status %d" % code)
        self.code = code


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            subprocess.run(["make", "-C", HERE, "oracle"], check=True, stdout=subprocess.DEVNULL)
        lib = ctypes.CDLL(LIB)
        vp, sz, u64, i32 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint64, ctypes.c_int
        lib.pskv_oracle_server_ranges.argtypes = [u64, vp, vp]
        lib.pskv_oracle_server_ranges.restype = None
        lib.pskv_oracle_slice.argtypes = [vp, sz, vp, sz, sz, vp, vp, sz, vp, vp, vp]
        lib.pskv_oracle_store_create.argtypes = [i32, u64]
        lib.pskv_oracle_store_create.restype = vp
        lib.pskv_oracle_store_destroy.argtypes = [vp]
        lib.pskv_oracle_store_destroy.restype = None
        lib.pskv_oracle_handle.argtypes = [vp, i32, i32, vp, sz, vp, sz, vp, sz, vp, sz, vp,
                                           ctypes.POINTER(sz)]
        lib.pskv_oracle_store_size.argtypes = [vp]
        lib.pskv_oracle_store_size.restype = sz
        lib.pskv_oracle_store_nvals.argtypes = [vp]
        lib.pskv_oracle_store_nvals.restype = sz
        lib.pskv_oracle_store_dump.argtypes = [vp, vp, vp, sz, vp, sz, ctypes.POINTER(sz),
                                               ctypes.POINTER(sz)]
        lib.pskv_oracle_assemble_pull.argtypes = [vp, sz, sz, vp, vp, vp, vp, vp, vp, sz, vp,
                                                  ctypes.POINTER(sz)]
        lib.pskv_oracle_find_range.argtypes = [vp, sz, u64, u64, ctypes.POINTER(u64),
                                               ctypes.POINTER(u64)]
        lib.pskv_oracle_find_range.restype = None
        lib.pskv_oracle_ordered_match.argtypes = [vp, sz, vp, vp, sz, vp, sz, ctypes.c_int,
                                                  ctypes.POINTER(sz)]
        _lib = lib
    return _lib


def have_ref():
    return os.path.exists(REF_LIB)


def load_ref():
    """The reference's own DefaultSlicer / FindRange (built by oracle/Makefile where the
    reference tree is present)."""
    global _ref
    if _ref is None:
        lib = ctypes.CDLL(REF_LIB)
        vp, sz, u64 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint64
        lib.pskv_ref_default_slicer.argtypes = [vp, sz, vp, sz, sz, vp, vp, sz, vp, vp, vp, vp, vp,
                                                ctypes.c_char_p, sz]
        lib.pskv_ref_find_range.argtypes = [vp, sz, u64, u64, ctypes.POINTER(u64),
                                            ctypes.POINTER(u64)]
        lib.pskv_ref_find_range.restype = None
        _ref = lib
    return _ref


def _p(a):
    return a.ctypes.data if a is not None and a.size else None


def _u64(a):
    return np.ascontiguousarray(a, dtype=np.uint64)


def server_ranges(S):
    b = np.zeros(S, np.uint64)
    e = np.zeros(S, np.uint64)
    load().pskv_oracle_server_ranges(S, b.ctypes.data, e.ctypes.data)
    return b, e


def slice_status(keys, range_begin, range_end, lens=None, nvals=0):
    """(status, pos, val_pos, used)"""
    keys = _u64(keys)
    rb, re = _u64(range_begin), _u64(range_end)
    S = rb.size
    lens_a = None if lens is None else np.ascontiguousarray(lens, dtype=np.int32)
    pos = np.zeros(S + 1, np.uint64)
    val_pos = np.zeros(S + 1, np.uint64)
    used = np.zeros(max(S, 1), np.uint8)
    rc = load().pskv_oracle_slice(_p(keys), keys.size, _p(lens_a),
                                  0 if lens_a is None else lens_a.size, nvals, _p(rb), _p(re), S,
                                  pos.ctypes.data, val_pos.ctypes.data, used.ctypes.data)
    return rc, pos, val_pos, used[:S]


def slice_keys(keys, range_begin, range_end, lens=None, nvals=0):
    rc, pos, val_pos, used = slice_status(keys, range_begin, range_end, lens, nvals)
    if rc != OK:
        raise OracleError(rc)
    return pos, val_pos, used


def ref_slice(keys, range_begin, range_end, lens=None, nvals=0):
    """Runs the reference's DefaultSlicer. Returns (ok, key_lo, key_hi, val_lo, val_hi, used, err)."""
    keys = _u64(keys)
    rb, re = _u64(range_begin), _u64(range_end)
    S = rb.size
    lens_a = None if lens is None else np.ascontiguousarray(lens, dtype=np.int32)
    outs = [np.zeros(max(S, 1), np.uint64) for _ in range(4)]
    used = np.zeros(max(S, 1), np.uint8)
    err = ctypes.create_string_buffer(1024)
    rc = load_ref().pskv_ref_default_slicer(_p(keys), keys.size, _p(lens_a),
                                            0 if lens_a is None else lens_a.size, nvals, _p(rb),
                                            _p(re), S, outs[0].ctypes.data, outs[1].ctypes.data,
                                            outs[2].ctypes.data, outs[3].ctypes.data,
                                            used.ctypes.data, err, 1024)
    return (rc == 0, outs[0][:S], outs[1][:S], outs[2][:S], outs[3][:S], used[:S],
            err.value.decode(errors="replace"))


def find_range(arr, lower, upper, use_ref=False):
    arr = _u64(arr)
    b, e = ctypes.c_uint64(0), ctypes.c_uint64(0)
    fn = load_ref().pskv_ref_find_range if use_ref else load().pskv_oracle_find_range
    fn(_p(arr), arr.size, lower, upper, ctypes.byref(b), ctypes.byref(e))
    return b.value, e.value


class Store:
    """The store of a request handle and one call per request (kv_app.h:440-463)."""

    def __init__(self, mode=MODE_SCALAR, row_len=0):
        self._lib = load()
        self._h = self._lib.pskv_oracle_store_create(mode, row_len)
        assert self._h
        self.mode = mode

    def __del__(self):
        try:
            if self._h:
                self._lib.pskv_oracle_store_destroy(self._h)
                self._h = None
        except Exception:
            pass

    def handle(self, push, pull, keys, vals=None, lens=None, out_cap=None):
        """Returns (status, out_vals, out_lens, out_nvals)."""
        keys = _u64(keys)
        n = keys.size
        vals_a = None if vals is None else np.ascontiguousarray(vals, dtype=np.float32)
        lens_a = None if lens is None else np.ascontiguousarray(lens, dtype=np.int32)
        got = ctypes.c_size_t(0)
        out = None
        out_lens = np.zeros(n, np.int32) if pull else None
        if pull and out_cap is None:
            # ask for the size first; the store is updated by this call, and the second
            # call below only reads rows that now exist
            rc = self._lib.pskv_oracle_handle(self._h, int(push), 1, _p(keys), n, _p(vals_a),
                                              0 if vals_a is None else vals_a.size, _p(lens_a),
                                              0 if lens_a is None else lens_a.size, None, 0,
                                              _p(out_lens), ctypes.byref(got))
            if rc not in (OK, ESIZE_MISMATCH) or (rc == ESIZE_MISMATCH and got.value == 0):
                return rc, None, None, got.value
            out = np.zeros(got.value, np.float32)
            rc = self._lib.pskv_oracle_handle(self._h, 0, 1, _p(keys), n, None, 0, None, 0, _p(out),
                                              out.size, _p(out_lens), ctypes.byref(got))
            return rc, out, out_lens, got.value
        if pull:
            out = np.zeros(out_cap, np.float32)
        rc = self._lib.pskv_oracle_handle(self._h, int(push), int(pull), _p(keys), n, _p(vals_a),
                                          0 if vals_a is None else vals_a.size, _p(lens_a),
                                          0 if lens_a is None else lens_a.size,
                                          None if out is None else _p(out),
                                          0 if out is None else out.size,
                                          None if out_lens is None else _p(out_lens),
                                          ctypes.byref(got))
        return rc, out, out_lens, got.value

    def push(self, keys, vals, lens=None):
        rc, _, _, _ = self.handle(True, False, keys, vals, lens)
        if rc != OK:
            raise OracleError(rc)

    def pull(self, keys):
        rc, out, out_lens, _ = self.handle(False, True, keys)
        if rc != OK:
            raise OracleError(rc)
        return out, out_lens

    def pushpull(self, keys, vals, lens=None):
        rc, out, out_lens, _ = self.handle(True, True, keys, vals, lens)
        if rc != OK:
            raise OracleError(rc)
        return out, out_lens

    def size(self):
        return self._lib.pskv_oracle_store_size(self._h), self._lib.pskv_oracle_store_nvals(self._h)

    def dump(self):
        nk, nv = self.size()
        keys = np.zeros(nk, np.uint64)
        lens = np.zeros(nk, np.int32)
        vals = np.zeros(nv, np.float32)
        a, b = ctypes.c_size_t(0), ctypes.c_size_t(0)
        rc = self._lib.pskv_oracle_store_dump(self._h, _p(keys), _p(lens), nk, _p(vals), nv,
                                              ctypes.byref(a), ctypes.byref(b))
        if rc != OK:
            raise OracleError(rc)
        return keys, lens, vals


def assemble_pull(req_keys, responses, want_lens=False):
    """responses: list of (keys, vals, lens-or-None) numpy arrays. Returns (status, vals, lens)."""
    req = _u64(req_keys)
    R = len(responses)
    PA = ctypes.c_void_p * max(R, 1)
    SA = ctypes.c_size_t * max(R, 1)
    kptr, vptr, lptr, nk, nv = PA(), PA(), PA(), SA(), SA()
    keep = []
    for i, (k, v, l) in enumerate(responses):
        k = _u64(k)
        v = np.ascontiguousarray(v, dtype=np.float32)
        keep += [k, v]
        kptr[i], nk[i], vptr[i], nv[i] = _p(k), k.size, _p(v), v.size
        if want_lens:
            l = np.ascontiguousarray(l, dtype=np.int32)
            keep.append(l)
            lptr[i] = _p(l)
    total = sum(int(x) for x in nv[:R])
    out = np.zeros(total, np.float32)
    out_lens = np.zeros(req.size, np.int32) if want_lens else None
    got = ctypes.c_size_t(0)
    rc = load().pskv_oracle_assemble_pull(_p(req), req.size, R, kptr, nk, vptr, nv,
                                          lptr if want_lens else None, _p(out), out.size,
                                          None if out_lens is None else _p(out_lens),
                                          ctypes.byref(got))
    return rc, out, out_lens


OP_ASSIGN, OP_PLUS, OP_MINUS, OP_TIMES, OP_DIVIDE = range(5)


def ordered_match(src_keys, src_vals, dst_keys, dst_vals, k=1, op=OP_ASSIGN):
    """ParallelOrderedMatch: returns (status, new dst_vals, matched values)."""
    sk, dk = _u64(src_keys), _u64(dst_keys)
    sv = np.ascontiguousarray(src_vals, dtype=np.float32)
    dv = np.array(dst_vals, dtype=np.float32, copy=True)
    assert sv.size == sk.size * k and dv.size == dk.size * k
    got = ctypes.c_size_t(0)
    rc = load().pskv_oracle_ordered_match(_p(sk), sk.size, _p(sv), _p(dk), dk.size, _p(dv), k, op,
                                          ctypes.byref(got))
    return rc, dv, got.value
