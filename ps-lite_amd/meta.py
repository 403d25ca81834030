"""ctypes binding of the message-header codec (include/pskv/meta_codec.h): the bytes of
Van::PackMeta / Van::UnpackMeta (src/van.cc:477-557) without protobuf.

A header is a dict:
  head, customer_id, priority, data_size: int      app_id, timestamp: int or None (unset)
  request, push, pull, simple_app: bool            body: bytes      data_type: list of int
  control: None or {cmd, barrier_group, msg_sig, nodes: [{role, id (int or None), port,
           customer_id, is_recovery, hostname: bytes}]}
"""
import ctypes

from . import capi

EMPTY = 2147483647  # Meta::kEmpty / Node::kEmpty
CTRL_EMPTY, CTRL_TERMINATE, CTRL_ADD_NODE, CTRL_BARRIER, CTRL_ACK, CTRL_HEARTBEAT = range(6)


class Node(ctypes.Structure):
    _fields_ = [("role", ctypes.c_int32), ("id", ctypes.c_int32), ("port", ctypes.c_int32),
                ("customer_id", ctypes.c_int32), ("is_recovery", ctypes.c_int32),
                ("hostname", ctypes.c_void_p), ("hostname_len", ctypes.c_size_t)]


class Meta(ctypes.Structure):
    _fields_ = [("head", ctypes.c_int32), ("app_id", ctypes.c_int32), ("customer_id", ctypes.c_int32),
                ("timestamp", ctypes.c_int32), ("request", ctypes.c_int32), ("push", ctypes.c_int32),
                ("pull", ctypes.c_int32), ("simple_app", ctypes.c_int32),
                ("body", ctypes.c_void_p), ("body_len", ctypes.c_size_t),
                ("data_type", ctypes.c_void_p), ("n_data_type", ctypes.c_size_t),
                ("control_cmd", ctypes.c_int32), ("has_control", ctypes.c_int32),
                ("barrier_group", ctypes.c_int32), ("msg_sig", ctypes.c_uint64),
                ("nodes", ctypes.c_void_p), ("n_nodes", ctypes.c_size_t),
                ("data_size", ctypes.c_int32), ("priority", ctypes.c_int32)]


_ready = False


def _lib():
    global _ready
    lib = capi.load()
    if not _ready:
        lib.pskv_meta_pack.argtypes = [ctypes.POINTER(Meta), ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t,
                                       ctypes.POINTER(ctypes.c_size_t)]
        lib.pskv_meta_unpack.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.POINTER(Meta),
                                         ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_size_t]
        _ready = True
    return lib


def pack(h, with_data_size=False):
    """The bytes Van::PackMeta writes for header `h` (Van::PackMetaPB with with_data_size)."""
    keep = []  # buffers the struct points into

    def buf(b):
        b = ctypes.create_string_buffer(bytes(b), len(b)) if len(b) else None
        keep.append(b)
        return ctypes.cast(b, ctypes.c_void_p) if b is not None else None

    m = Meta()
    m.head, m.customer_id = h["head"], h.get("customer_id", 0)
    m.app_id = EMPTY if h.get("app_id") is None else h["app_id"]
    m.timestamp = EMPTY if h.get("timestamp") is None else h["timestamp"]
    m.request, m.push, m.pull, m.simple_app = (int(bool(h.get(k, False))) for k in
                                               ("request", "push", "pull", "simple_app"))
    body = h.get("body", b"")
    m.body, m.body_len = buf(body), len(body)
    types = list(h.get("data_type", []))
    arr = (ctypes.c_int32 * max(len(types), 1))(*types)
    keep.append(arr)
    m.data_type, m.n_data_type = ctypes.cast(arr, ctypes.c_void_p), len(types)
    c = h.get("control")
    m.control_cmd = CTRL_EMPTY if c is None else c["cmd"]
    if c is not None:
        m.barrier_group, m.msg_sig = c.get("barrier_group", 0), c.get("msg_sig", 0)
        nodes = c.get("nodes", [])
        narr = (Node * max(len(nodes), 1))()
        for i, n in enumerate(nodes):
            narr[i].role, narr[i].port, narr[i].customer_id = n["role"], n.get("port", 0), n.get("customer_id", 0)
            narr[i].id = EMPTY if n.get("id") is None else n["id"]
            narr[i].is_recovery = int(bool(n.get("is_recovery", False)))
            hn = n.get("hostname", b"")
            narr[i].hostname, narr[i].hostname_len = buf(hn), len(hn)
        keep.append(narr)
        m.nodes, m.n_nodes = ctypes.cast(narr, ctypes.c_void_p), len(nodes)
    m.data_size, m.priority = h.get("data_size", 0), h.get("priority", 0)
    need = ctypes.c_size_t(0)
    _lib().pskv_meta_pack(ctypes.byref(m), int(with_data_size), None, 0, ctypes.byref(need))
    out = ctypes.create_string_buffer(max(need.value, 1))
    rc = _lib().pskv_meta_pack(ctypes.byref(m), int(with_data_size), out, need.value, ctypes.byref(need))
    if rc != 0:
        raise capi.PskvError(rc, "pskv_meta_pack")
    return out.raw[:need.value]


def unpack(data):
    """The header Van::UnpackMeta reads from `data`; raises PskvError(EINVAL) for bytes that are
    not a PBMeta."""
    data = bytes(data)
    src = ctypes.create_string_buffer(data, max(len(data), 1))
    m = Meta()
    ncap, tcap = 8, 16
    while True:
        nodes = (Node * ncap)()
        types = (ctypes.c_int32 * tcap)()
        rc = _lib().pskv_meta_unpack(src, len(data), ctypes.byref(m), nodes, ncap, types, tcap)
        if rc == capi.ESIZE_MISMATCH:
            ncap, tcap = max(ncap, m.n_nodes), max(tcap, m.n_data_type)
            continue
        break
    if rc != 0:
        raise capi.PskvError(rc, "not a message header")

    def view(ptr, n):
        return ctypes.string_at(ptr, n) if ptr and n else b""

    h = {"head": m.head, "app_id": None if m.app_id == EMPTY else m.app_id, "customer_id": m.customer_id,
         "timestamp": None if m.timestamp == EMPTY else m.timestamp, "request": bool(m.request),
         "push": bool(m.push), "pull": bool(m.pull), "simple_app": bool(m.simple_app),
         "body": view(m.body, m.body_len), "data_type": [types[i] for i in range(m.n_data_type)],
         "data_size": m.data_size, "priority": m.priority, "control": None}
    if m.has_control:
        h["control"] = {"cmd": m.control_cmd, "barrier_group": m.barrier_group, "msg_sig": m.msg_sig,
                        "nodes": [{"role": nodes[i].role, "id": None if nodes[i].id == EMPTY else nodes[i].id,
                                   "port": nodes[i].port, "customer_id": nodes[i].customer_id,
                                   "is_recovery": bool(nodes[i].is_recovery),
                                   "hostname": view(nodes[i].hostname, nodes[i].hostname_len)}
                                  for i in range(m.n_nodes)]}
    return h
