"""ctypes binding of libpskv.so, the C ABI declared in include/pskv/capi.h.

Buffers are either numpy arrays (host memory, PSKV_MEM_HOST) or torch tensors
on the table's device (PSKV_MEM_DEVICE). torch is only the owner of device
memory here; every computation happens inside libpskv.so.
"""
import ctypes
import os
import sys
import weakref

import numpy as np

from . import build as _build

OK = 0
EUNCOVERED_KEY = -1
ESIZE_MISMATCH = -2
ENOMEM = -3
EHIP = -4
EINVAL = -5
ERANGE_GAP = -6
ELEN_CHANGED = -7
ESTALE = -8
REPLAY_PUSH = 1
REPLAY_PULL = 2
REPLAY_LAUNCHES = 4
MEM_HOST = 0
MEM_DEVICE = 1
MODE_SCALAR = 0
MODE_FIXED = 1
MODE_VARLEN = 2
MAX_VARLEN_ROW = (1 << 28) - 1
SLICE_NOALLOC_MAX_RANGES = 1024
KERNEL_PUSH_SCALAR, KERNEL_PULL_SCALAR, KERNEL_ROWS_ACC, KERNEL_ROWS_GATHER, KERNEL_LOOKUP, \
    KERNEL_REHASH, KERNEL_COPY, KERNEL_SAME_KEYS, KERNEL_PULL_PER_KEY = range(9)

ERROR_NAMES = {
    EUNCOVERED_KEY: "PSKV_EUNCOVERED_KEY", ESIZE_MISMATCH: "PSKV_ESIZE_MISMATCH",
    ENOMEM: "PSKV_ENOMEM", EHIP: "PSKV_EHIP", EINVAL: "PSKV_EINVAL",
    ERANGE_GAP: "PSKV_ERANGE_GAP", ELEN_CHANGED: "PSKV_ELEN_CHANGED", ESTALE: "PSKV_ESTALE",
}

# every symbol include/pskv/capi.h declares
SYMBOLS = [
    "pskv_table_create", "pskv_table_destroy", "pskv_push", "pskv_pull", "pskv_pushpull",
    "pskv_sync", "pskv_table_stream", "pskv_push_multi", "pskv_pull_multi", "pskv_pushpull_multi", "pskv_sync_multi", "pskv_replay_record", "pskv_replay_run", "pskv_replay_destroy", "pskv_size", "pskv_dump", "pskv_slice", "pskv_slice_noalloc", "pskv_server_ranges",
    "pskv_assemble_pull", "pskv_match", "pskv_prof_enable", "pskv_prof_reset", "pskv_prof_read", "pskv_prof_samples",
    "pskv_copy_probe", "pskv_host_alloc", "pskv_host_free", "pskv_host_trim", "pskv_device_trim", "pskv_table_counters", "pskv_last_error",
    "pskv_version",
]


class PskvError(RuntimeError):
    def __init__(self, code, text):
        super().__init__("%s: %s" % (ERROR_NAMES.get(code, code), text))
        self.code = code


class Opts(ctypes.Structure):
    _fields_ = [
        ("device", ctypes.c_int32), ("mode", ctypes.c_int32),
        ("initial_capacity", ctypes.c_uint64), ("row_len", ctypes.c_uint64),
        ("arena_floats", ctypes.c_uint64), ("max_load", ctypes.c_float),
        ("reserved", ctypes.c_uint32), ("stream", ctypes.c_void_p),
    ]


_lib = None


def load():
    """Loads the built library. There is no fallback: a missing library is an error."""
    global _lib
    if _lib is not None:
        return _lib
    path = _build.lib_path()
    if not os.path.exists(path):
        raise RuntimeError(
            "libpskv.so is not built (%s); run `python -c 'import __graft_entry__ as g; g.build()'`" % path)
    try:
        import torch  # noqa: F401  (so that one HIP runtime serves torch and this library)
    except ImportError:
        pass
    lib = ctypes.CDLL(path)
    vp, sz, i32, u64 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_uint64
    lib.pskv_table_create.argtypes = [ctypes.POINTER(vp), ctypes.POINTER(Opts)]
    lib.pskv_table_destroy.argtypes = [vp]
    lib.pskv_push.argtypes = [vp, vp, sz, vp, sz, vp, sz, i32]
    lib.pskv_pull.argtypes = [vp, vp, sz, vp, sz, vp, ctypes.POINTER(sz), i32]
    lib.pskv_pushpull.argtypes = [vp, vp, sz, vp, sz, vp, sz, vp, sz, vp, ctypes.POINTER(sz), i32]
    lib.pskv_sync.argtypes = [vp]
    lib.pskv_table_stream.argtypes = [vp]
    lib.pskv_table_stream.restype = vp
    lib.pskv_push_multi.argtypes = [vp, sz, vp, vp, vp, vp, vp, i32]
    lib.pskv_pull_multi.argtypes = [vp, sz, vp, vp, vp, vp, vp, vp, i32]
    lib.pskv_pushpull_multi.argtypes = [vp, sz, vp, vp, vp, vp, vp, vp, vp, vp, vp, i32]
    lib.pskv_sync_multi.argtypes = [vp, sz]
    lib.pskv_replay_record.argtypes = [ctypes.POINTER(vp), vp, sz, i32, vp, vp, vp, vp, vp, vp, vp, vp]
    lib.pskv_replay_run.argtypes = [vp]
    lib.pskv_replay_destroy.argtypes = [vp]
    lib.pskv_size.argtypes = [vp, ctypes.POINTER(u64), ctypes.POINTER(u64)]
    lib.pskv_dump.argtypes = [vp, vp, vp, sz, vp, sz, ctypes.POINTER(sz), ctypes.POINTER(sz)]
    lib.pskv_slice.argtypes = [i32, vp, sz, vp, sz, sz, vp, vp, sz, vp, vp, vp, i32]
    lib.pskv_slice_noalloc.argtypes = [i32, vp, vp, sz, vp, sz, sz, vp, vp, sz, vp, vp, vp, vp]
    lib.pskv_server_ranges.argtypes = [u64, vp, vp]
    lib.pskv_assemble_pull.argtypes = [i32, vp, sz, sz, vp, vp, vp, vp, vp, vp, sz, vp,
                                       ctypes.POINTER(sz), i32]
    lib.pskv_match.argtypes = [i32, vp, sz, vp, vp, sz, vp, sz, i32, ctypes.POINTER(u64), vp, i32]
    lib.pskv_prof_enable.argtypes = [vp, i32]
    lib.pskv_prof_reset.argtypes = [vp]
    lib.pskv_prof_read.argtypes = [vp, i32, ctypes.POINTER(u64), ctypes.POINTER(ctypes.c_double)]
    lib.pskv_prof_samples.argtypes = [vp, i32, vp, sz, ctypes.POINTER(sz)]
    lib.pskv_copy_probe.argtypes = [vp, vp, vp, sz]
    lib.pskv_host_alloc.argtypes = [sz]
    lib.pskv_host_alloc.restype = vp
    lib.pskv_host_free.argtypes = [vp]
    lib.pskv_host_free.restype = None
    lib.pskv_device_trim.argtypes = [i32]
    lib.pskv_table_counters.argtypes = [vp, vp, sz]
    lib.pskv_last_error.restype = ctypes.c_char_p
    lib.pskv_version.restype = ctypes.c_char_p
    _lib = lib
    return lib


def _check(rc):
    if rc != OK:
        raise PskvError(rc, load().pskv_last_error().decode())


def _is_tensor(x):
    return hasattr(x, "data_ptr")


def _buf(x, dtype_np, dtype_name):
    """(pointer, element count, memkind or None) of a numpy array / torch tensor / None."""
    if x is None:
        return None, 0, None
    if _is_tensor(x):
        assert str(x.dtype).endswith(dtype_name), (x.dtype, dtype_name)
        assert x.is_contiguous()
        kind = MEM_DEVICE if x.is_cuda else MEM_HOST
        return (x.data_ptr() if x.numel() else None), x.numel(), kind
    a = np.ascontiguousarray(x, dtype=dtype_np)
    return (a.ctypes.data if a.size else None), a.size, MEM_HOST


def _memkind(*kinds):
    ks = {k for k in kinds if k is not None}
    assert len(ks) <= 1, "all buffers of a call must live in the same kind of memory"
    kind = ks.pop() if ks else MEM_HOST
    if kind == MEM_DEVICE:
        # The C ABI wants device buffers complete before the call (the library runs on streams of
        # its own). torch fills and copies tensors asynchronously on ITS current stream, so the
        # methods that take tensors wait for that stream first; the *_raw methods leave it to
        # the caller.
        import torch
        torch.cuda.current_stream().synchronize()
    return kind


class _Holder:
    """Device-resident calls are asynchronous: the table reads and writes the caller's tensors after
    the call has returned. The methods that take tensors therefore keep them referenced until the
    next wait, so that a temporary (`t.push(to_dev(keys), ...)`) is not handed to someone else by
    torch's allocator while a kernel is still to read it. The *_raw methods leave that to the caller."""

    def _hold(self, *tensors):
        held = self.__dict__.setdefault("_held", [])
        held.extend(x for x in tensors if x is not None and _is_tensor(x) and x.is_cuda)
        if len(held) > 4096:
            self.sync()

    def _release(self):
        self.__dict__["_held"] = []


class Table(_Holder):
    """The store behind a KVServer request handle (kv_app.h:440-463)."""

    def __init__(self, mode=MODE_SCALAR, device=0, initial_capacity=0, row_len=0, arena_floats=0,
                 max_load=0.0, stream=None):
        self._lib = load()
        self._h = ctypes.c_void_p()
        o = Opts(device, mode, initial_capacity, row_len, arena_floats, max_load, 0, stream)
        _check(self._lib.pskv_table_create(ctypes.byref(self._h), ctypes.byref(o)))
        self.mode = mode
        self.device = device

    def close(self):
        if self._h:
            self._lib.pskv_table_destroy(self._h)
            self._h = ctypes.c_void_p()
        self._release()

    def __del__(self):
        # Not while the interpreter shuts down: a stream that the caller lent (torch's, say) may be
        # gone by then, and the process is about to give everything back anyway.
        if sys is None or sys.is_finalizing():
            return
        try:
            self.close()
        except Exception:
            pass

    def push(self, keys, vals, lens=None):
        kp, n, k1 = _buf(keys, np.uint64, "int64")
        vp, nv, k2 = _buf(vals, np.float32, "float32")
        lp, nl, k3 = _buf(lens, np.int32, "int32")
        self._hold(keys, vals, lens)
        _check(self._lib.pskv_push(self._h, kp, n, vp, nv, lp, nl, _memkind(k1, k2, k3)))

    def pull(self, keys, out, out_lens=None):
        """Returns the number of floats of the response."""
        kp, n, k1 = _buf(keys, np.uint64, "int64")
        op, cap, k2 = _buf(out, np.float32, "float32")
        lp, _, k3 = _buf(out_lens, np.int32, "int32")
        got = ctypes.c_size_t(0)
        self.last_out_nvals = None
        self._hold(keys, out, out_lens)
        rc = self._lib.pskv_pull(self._h, kp, n, op, cap, lp, ctypes.byref(got), _memkind(k1, k2, k3))
        self.last_out_nvals = got.value
        _check(rc)
        return got.value

    def pushpull(self, keys, vals, out, lens=None, out_lens=None):
        kp, n, k1 = _buf(keys, np.uint64, "int64")
        vp, nv, k2 = _buf(vals, np.float32, "float32")
        lp, nl, k3 = _buf(lens, np.int32, "int32")
        op, cap, k4 = _buf(out, np.float32, "float32")
        olp, _, k5 = _buf(out_lens, np.int32, "int32")
        got = ctypes.c_size_t(0)
        self._hold(keys, vals, lens, out, out_lens)
        rc = self._lib.pskv_pushpull(self._h, kp, n, vp, nv, lp, nl, op, cap, olp, ctypes.byref(got),
                                     _memkind(k1, k2, k3, k4, k5))
        self.last_out_nvals = got.value
        _check(rc)
        return got.value

    def push_raw(self, keys_ptr, n, vals_ptr, nvals, lens_ptr=None, nlens=0):
        """pskv_push on raw device addresses (no per-call tensor bookkeeping)."""
        _check(self._lib.pskv_push(self._h, keys_ptr, n, vals_ptr, nvals, lens_ptr, nlens, MEM_DEVICE))

    def pull_raw(self, keys_ptr, n, out_ptr, out_cap, out_lens_ptr=None):
        _check(self._lib.pskv_pull(self._h, keys_ptr, n, out_ptr, out_cap, out_lens_ptr, None,
                                   MEM_DEVICE))

    def pushpull_raw(self, keys_ptr, n, vals_ptr, nvals, out_ptr, out_cap):
        """pskv_pushpull (one request with both halves) on raw device addresses, SCALAR / FIXED tables."""
        _check(self._lib.pskv_pushpull(self._h, keys_ptr, n, vals_ptr, nvals, None, 0, out_ptr, out_cap, None, None,
                                       MEM_DEVICE))

    def sync(self):
        rc = self._lib.pskv_sync(self._h)
        self._release()
        _check(rc)

    def size(self):
        nk, nv = ctypes.c_uint64(0), ctypes.c_uint64(0)
        _check(self._lib.pskv_size(self._h, ctypes.byref(nk), ctypes.byref(nv)))
        return nk.value, nv.value

    def counters(self):
        """What the table's sizing logic has done so far, by name (pskv_table_counters)."""
        out = np.zeros(8, np.uint64)
        _check(self._lib.pskv_table_counters(self._h, out.ctypes.data, out.size))
        names = ("requests", "growths", "growths_unasked", "growths_ahead", "waits", "catch_ups", "records", "slots")
        return {k: int(v) for k, v in zip(names, out)}

    def dump(self):
        """(keys sorted, lens, vals) as numpy arrays."""
        nk, nv = self.size()
        keys = np.zeros(nk, np.uint64)
        lens = np.zeros(nk, np.int32)
        vals = np.zeros(nv, np.float32)
        a, b = ctypes.c_size_t(0), ctypes.c_size_t(0)
        _check(self._lib.pskv_dump(self._h, keys.ctypes.data, lens.ctypes.data, nk, vals.ctypes.data,
                                   nv, ctypes.byref(a), ctypes.byref(b)))
        return keys, lens, vals

    def prof_enable(self, on=True):
        _check(self._lib.pskv_prof_enable(self._h, 1 if on else 0))

    def prof_reset(self):
        _check(self._lib.pskv_prof_reset(self._h))

    def prof_read(self, kernel):
        n, ms = ctypes.c_uint64(0), ctypes.c_double(0.0)
        _check(self._lib.pskv_prof_read(self._h, kernel, ctypes.byref(n), ctypes.byref(ms)))
        return n.value, ms.value

    def prof_samples(self, kernel):
        """Durations (ms) of the individual launches since the last prof_reset."""
        n = ctypes.c_size_t(0)
        _check(self._lib.pskv_prof_samples(self._h, kernel, None, 0, ctypes.byref(n)))
        out = np.zeros(n.value, np.float32)
        if n.value:
            _check(self._lib.pskv_prof_samples(self._h, kernel, out.ctypes.data, out.size, ctypes.byref(n)))
        return out

    def copy_probe(self, dst, src):
        assert dst.is_cuda and src.is_cuda
        _memkind(MEM_DEVICE)  # (torch may still be filling the tensors on its own stream)
        self._hold(dst, src)
        nbytes = src.numel() * src.element_size()
        _check(self._lib.pskv_copy_probe(self._h, dst.data_ptr(), src.data_ptr(), nbytes))


class Group(_Holder):
    """Several tables of one process on one GPU that share a stream, so that one launch per
    pipeline step serves all key ranges of a sliced request (pskv_push_multi / pskv_pull_multi)."""

    def __init__(self, S, mode=MODE_SCALAR, device=0, initial_capacity=0, row_len=0, arena_floats=0,
                 max_load=0.0, stream=None):
        self.tables = []
        for s in range(S):
            t = Table(mode, device, initial_capacity, row_len, arena_floats, max_load, stream)
            if stream is None:
                stream = load().pskv_table_stream(t._h)
            self.tables.append(t)
        self.S = S
        self.mode = mode
        self._arr = (ctypes.c_void_p * max(S, 1))(*[t._h for t in self.tables])
        self._lib = load()

    def close(self):
        # recordings go before the tables they point at
        for ref in self.__dict__.get("_recordings", []):
            rec = ref()
            if rec is not None:
                rec.close()
        self.__dict__["_recordings"] = []
        # the first table owns the stream the others run on: it goes last
        for t in reversed(self.tables):
            t.close()
        self.tables = []

    def __del__(self):
        # Not while the interpreter shuts down: a stream that the caller lent (torch's, say) may be
        # gone by then, and the process is about to give everything back anyway.
        if sys is None or sys.is_finalizing():
            return
        try:
            self.close()
        except Exception:
            pass

    def push_raw(self, keys_ptr, pos, vals_ptr, val_pos, lens_ptr=None):
        """pos / val_pos: numpy uint64 arrays of S+1 entries as pskv_slice returns them."""
        pos = np.ascontiguousarray(pos, dtype=np.uint64)
        val_pos = np.ascontiguousarray(val_pos, dtype=np.uint64)
        _check(self._lib.pskv_push_multi(self._arr, self.S, keys_ptr, pos.ctypes.data, vals_ptr,
                                         val_pos.ctypes.data, lens_ptr, MEM_DEVICE))

    def pull_raw(self, keys_ptr, pos, out_ptr, out_pos=None, out_lens_ptr=None, want_sizes=False):
        """Returns the per-slice response sizes (numpy uint64) when want_sizes, else None."""
        pos = np.ascontiguousarray(pos, dtype=np.uint64)
        op = None
        if out_pos is not None:
            out_pos = np.ascontiguousarray(out_pos, dtype=np.uint64)
            op = out_pos.ctypes.data
        sizes = np.zeros(max(self.S, 1), np.uint64) if want_sizes else None
        rc = self._lib.pskv_pull_multi(self._arr, self.S, keys_ptr, pos.ctypes.data, out_ptr, op,
                                       out_lens_ptr, sizes.ctypes.data if want_sizes else None, MEM_DEVICE)
        self.last_sizes = sizes
        _check(rc)
        return sizes[:self.S] if want_sizes else None

    def pushpull_raw(self, keys_ptr, pos, vals_ptr, val_pos, out_ptr, out_pos=None, lens_ptr=None, out_lens_ptr=None):
        pos = np.ascontiguousarray(pos, dtype=np.uint64)
        val_pos = np.ascontiguousarray(val_pos, dtype=np.uint64)
        op = None if out_pos is None else np.ascontiguousarray(out_pos, dtype=np.uint64)
        _check(self._lib.pskv_pushpull_multi(self._arr, self.S, keys_ptr, pos.ctypes.data, vals_ptr,
                                             val_pos.ctypes.data, lens_ptr, out_ptr,
                                             None if op is None else op.ctypes.data, out_lens_ptr, None, MEM_DEVICE))

    def pushpull(self, keys, pos, vals, val_pos, out, lens=None, out_pos=None, out_lens=None, want_sizes=False):
        """pskv_pushpull_multi: one request with both halves over all slices."""
        _memkind(MEM_DEVICE)
        self._hold(keys, vals, lens, out, out_lens)
        pos = np.ascontiguousarray(pos, dtype=np.uint64)
        val_pos = np.ascontiguousarray(val_pos, dtype=np.uint64)
        op = None if out_pos is None else np.ascontiguousarray(out_pos, dtype=np.uint64)
        sizes = np.zeros(max(self.S, 1), np.uint64) if want_sizes else None

        def ptr(x):
            return None if x is None or not x.numel() else x.data_ptr()

        _check(self._lib.pskv_pushpull_multi(self._arr, self.S, ptr(keys), pos.ctypes.data, ptr(vals),
                                             val_pos.ctypes.data, ptr(lens), ptr(out),
                                             None if op is None else op.ctypes.data, ptr(out_lens),
                                             sizes.ctypes.data if want_sizes else None, MEM_DEVICE))
        return sizes[:self.S] if want_sizes else None

    def push(self, keys, pos, vals, val_pos, lens=None):
        _memkind(MEM_DEVICE)
        self._hold(keys, vals, lens)
        self.push_raw(keys.data_ptr() if keys.numel() else None, pos,
                      vals.data_ptr() if vals.numel() else None, val_pos,
                      None if lens is None else (lens.data_ptr() if lens.numel() else None))

    def pull(self, keys, pos, out, out_pos=None, out_lens=None, want_sizes=False):
        _memkind(MEM_DEVICE)
        self._hold(keys, out, out_lens)
        return self.pull_raw(keys.data_ptr() if keys.numel() else None, pos,
                             out.data_ptr() if out.numel() else None, out_pos,
                             None if out_lens is None else (out_lens.data_ptr() if out_lens.numel() else None),
                             want_sizes)

    def sync(self):
        rc = self._lib.pskv_sync_multi(self._arr, self.S)
        self._release()
        _check(rc)

    def record(self, what, keys, pos, vals=None, val_pos=None, lens=None, out=None, out_pos=None, out_lens=None):
        """pskv_replay_record: serves the request once and returns a Replay whose run() repeats it with
        one launch. The tensors are referenced by the Replay for as long as it lives."""
        _memkind(MEM_DEVICE)
        pos = np.ascontiguousarray(pos, dtype=np.uint64)
        vp = None if val_pos is None else np.ascontiguousarray(val_pos, dtype=np.uint64)
        op = None if out_pos is None else np.ascontiguousarray(out_pos, dtype=np.uint64)

        def ptr(x):
            return None if x is None or not x.numel() else x.data_ptr()

        h = ctypes.c_void_p()
        _check(self._lib.pskv_replay_record(ctypes.byref(h), self._arr, self.S, what, ptr(keys), pos.ctypes.data,
                                            ptr(vals), None if vp is None else vp.ctypes.data, ptr(lens), ptr(out),
                                            None if op is None else op.ctypes.data, ptr(out_lens)))
        rec = Replay(h, (keys, vals, lens, out, out_lens))
        self.__dict__.setdefault("_recordings", []).append(weakref.ref(rec))
        return rec

    def size(self):
        nk = nv = 0
        for t in self.tables:
            a, b = t.size()
            nk, nv = nk + a, nv + b
        return nk, nv


class Replay:
    """A recorded request (pskv_replay_*). Close it before the tables it was recorded on."""

    def __init__(self, handle, held):
        self._h = handle
        self._held = held
        self._lib = load()

    def run(self):
        _check(self._lib.pskv_replay_run(self._h))

    def close(self):
        if self._h:
            self._lib.pskv_replay_destroy(self._h)
            self._h = None
            self._held = None

    def __del__(self):
        if sys is None or sys.is_finalizing():
            return
        try:
            self.close()
        except Exception:
            pass


def server_ranges(num_servers):
    """Postoffice::GetServerKeyRanges (src/postoffice.cc:169-180) as two uint64 arrays."""
    b = np.zeros(num_servers, np.uint64)
    e = np.zeros(num_servers, np.uint64)
    _check(load().pskv_server_ranges(num_servers, b.ctypes.data, e.ctypes.data))
    return b, e


def slice_keys(keys, range_begin, range_end, lens=None, nvals=0, device=0):
    """KVWorker::DefaultSlicer (kv_app.h:517-572): returns (pos, val_pos, used)."""
    kp, n, k1 = _buf(keys, np.uint64, "int64")
    lp, nl, k2 = _buf(lens, np.int32, "int32")
    rb = np.ascontiguousarray(range_begin, dtype=np.uint64)
    re = np.ascontiguousarray(range_end, dtype=np.uint64)
    S = rb.size
    pos = np.zeros(S + 1, np.uint64)
    val_pos = np.zeros(S + 1, np.uint64)
    used = np.zeros(max(S, 1), np.uint8)
    _check(load().pskv_slice(device, kp, n, lp, nl, nvals, rb.ctypes.data, re.ctypes.data, S,
                             pos.ctypes.data, val_pos.ctypes.data, used.ctypes.data,
                             _memkind(k1, k2)))
    return pos, val_pos, used[:S]


def slice_keys_noalloc(keys, range_begin, range_end, pos, val_pos, used, status, lens=None, nvals=0,
                       device=0, stream=None):
    """pskv_slice_noalloc: device tensors in (keys int64, lens int32 or None) and out (pos and
    val_pos int64 of S+1, used uint8 of S, status int32 of 1); asynchronous on `stream`."""
    kp, n, _ = _buf(keys, np.uint64, "int64")
    lp, nl, _ = _buf(lens, np.int32, "int32")
    rb = np.ascontiguousarray(range_begin, dtype=np.uint64)
    re = np.ascontiguousarray(range_end, dtype=np.uint64)
    _memkind(MEM_DEVICE)  # (torch may still be filling the tensors on its own stream)
    _check(load().pskv_slice_noalloc(device, stream, kp, n, lp, nl, nvals, rb.ctypes.data,
                                     re.ctypes.data, rb.size, pos.data_ptr(), val_pos.data_ptr(),
                                     used.data_ptr(), status.data_ptr()))


def assemble_pull(req_keys, responses, out, out_lens=None, device=0):
    """Device-side counterpart of the KVWorker::AddPullCB callback (kv_app.h:663-714).
    responses: list of (keys, vals, lens-or-None) device tensors in arrival order."""
    R = len(responses)
    PA = ctypes.c_void_p * max(R, 1)
    SA = ctypes.c_size_t * max(R, 1)
    kptr, vptr, lptr, nk, nv = PA(), PA(), PA(), SA(), SA()
    have_lens = R > 0 and all(r[2] is not None for r in responses)
    for i, (k, v, l) in enumerate(responses):
        kptr[i], nk[i] = k.data_ptr() if k.numel() else None, k.numel()
        vptr[i], nv[i] = v.data_ptr() if v.numel() else None, v.numel()
        if have_lens:
            lptr[i] = l.data_ptr() if l.numel() else None
    kp, n, _ = _buf(req_keys, np.uint64, "int64")
    op, cap, _ = _buf(out, np.float32, "float32")
    olp, _, _ = _buf(out_lens, np.int32, "int32")
    got = ctypes.c_size_t(0)
    _memkind(MEM_DEVICE)  # (torch may still be filling the tensors on its own stream)
    _check(load().pskv_assemble_pull(device, kp, n, R, kptr, nk, vptr, nv,
                                     lptr if have_lens else None, op, cap, olp, ctypes.byref(got),
                                     MEM_DEVICE))
    return got.value


OP_ASSIGN, OP_PLUS, OP_MINUS, OP_TIMES, OP_DIVIDE = range(5)


def match(src_keys, src_vals, dst_keys, dst_vals, k=1, op=OP_ASSIGN, device=0, kernel_ms=None):
    """ParallelOrderedMatch (parallel_kv_match.h:29-120) on the GPU: dst_vals[i] op= src_vals[j] wherever
    dst_keys[i] == src_keys[j], in place. numpy arrays (host memory) or torch tensors on the device.
    Returns the number of matched VALUES (k per matched key). kernel_ms: None, or a float32 numpy array of
    two entries that receives the device time of the call's key kernel and row kernel."""
    skp, ns, m1 = _buf(src_keys, np.uint64, "int64")
    svp, nsv, m2 = _buf(src_vals, np.float32, "float32")
    dkp, nd, m3 = _buf(dst_keys, np.uint64, "int64")
    dvp, ndv, m4 = _buf(dst_vals, np.float32, "float32")
    assert nsv == ns * k and ndv == nd * k, "k values per key on both sides"
    if not _is_tensor(dst_vals):
        assert isinstance(dst_vals, np.ndarray) and dst_vals.dtype == np.float32 and \
            dst_vals.flags.c_contiguous, "dst_vals is changed in place"
    got = ctypes.c_uint64(0)
    _check(load().pskv_match(device, skp, ns, svp, dkp, nd, dvp, k, op, ctypes.byref(got),
                             None if kernel_ms is None else kernel_ms.ctypes.data, _memkind(m1, m2, m3, m4)))
    return got.value


def version():
    return load().pskv_version().decode()


def host_alloc(nbytes):
    """A pinned host buffer (address) from the library's pool; give it back with host_free."""
    p = load().pskv_host_alloc(nbytes)
    if not p:
        raise PskvError(ENOMEM, load().pskv_last_error().decode())
    return p


def host_free(ptr):
    load().pskv_host_free(ptr)


def host_trim():
    _check(load().pskv_host_trim())


def device_trim(device=0):
    """Gives the device memory that the library keeps for reuse back to the system."""
    _check(load().pskv_device_trim(device))


def host_array(ptr, count, dtype):
    """A numpy view of `count` elements of `dtype` at a pinned address from host_alloc."""
    dt = np.dtype(dtype)
    raw = (ctypes.c_char * (count * dt.itemsize)).from_address(ptr)
    return np.frombuffer(raw, dtype=dt, count=count)
