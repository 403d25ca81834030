"""Writes tests/golden/meta_golden.json: message headers and the bytes the protobuf runtime
serialises them to.

The reference packs ps::Meta through the generated class of src/meta.proto (Van::PackMeta,
src/van.cc:477-514). protoc and libprotobuf are not part of this image, but the protobuf
Python runtime is: the three messages of meta.proto are declared here field by field
(numbers, types, labels and the packed option as in src/meta.proto:8-60), filled the way
van.cc:480-507 fills them, and serialised by that runtime. The wire format does not depend on
the runtime's language or version. Run from the repository root:
    python tests/golden/make_meta_golden.py
"""
import json
import os
import sys

from google.protobuf import descriptor_pb2, descriptor_pool, message_factory
import google.protobuf

HERE = os.path.dirname(os.path.abspath(__file__))
EMPTY = 2147483647  # Meta::kEmpty, Node::kEmpty (src/customer.cc:8-9)
BARRIER, ACK = 3, 4  # Control::Command (include/ps/internal/message.h:101)
F = descriptor_pb2.FieldDescriptorProto


def pb_classes():
    fd = descriptor_pb2.FileDescriptorProto()
    fd.name, fd.package, fd.syntax = "ps_meta_for_golden.proto", "ps", "proto2"

    def msg(name, fields):
        m = fd.message_type.add()
        m.name = name
        for fname, number, ftype, label, extra in fields:
            f = m.field.add()
            f.name, f.number, f.type, f.label = fname, number, ftype, label
            if extra.get("type_name"):
                f.type_name = extra["type_name"]
            if extra.get("packed"):
                f.options.packed = True

    opt, req, rep = F.LABEL_OPTIONAL, F.LABEL_REQUIRED, F.LABEL_REPEATED
    msg("PBNode", [("role", 1, F.TYPE_INT32, req, {}), ("id", 2, F.TYPE_INT32, opt, {}),
                   ("hostname", 3, F.TYPE_STRING, opt, {}), ("port", 4, F.TYPE_INT32, opt, {}),
                   ("is_recovery", 5, F.TYPE_BOOL, opt, {}), ("customer_id", 10, F.TYPE_INT32, opt, {})])
    msg("PBControl", [("cmd", 1, F.TYPE_INT32, req, {}),
                      ("node", 2, F.TYPE_MESSAGE, rep, {"type_name": ".ps.PBNode"}),
                      ("barrier_group", 3, F.TYPE_INT32, opt, {}), ("msg_sig", 4, F.TYPE_UINT64, opt, {})])
    msg("PBMeta", [("head", 1, F.TYPE_INT32, opt, {}), ("body", 2, F.TYPE_BYTES, opt, {}),
                   ("control", 3, F.TYPE_MESSAGE, opt, {"type_name": ".ps.PBControl"}),
                   ("request", 4, F.TYPE_BOOL, opt, {}), ("app_id", 7, F.TYPE_INT32, opt, {}),
                   ("timestamp", 8, F.TYPE_INT32, opt, {}),
                   ("data_type", 9, F.TYPE_INT32, rep, {"packed": True}),
                   ("customer_id", 10, F.TYPE_INT32, opt, {}), ("push", 5, F.TYPE_BOOL, opt, {}),
                   ("pull", 12, F.TYPE_BOOL, opt, {}), ("simple_app", 6, F.TYPE_BOOL, opt, {}),
                   ("data_size", 11, F.TYPE_INT32, opt, {}), ("priority", 13, F.TYPE_INT32, opt, {})])
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    get = getattr(message_factory, "GetMessageClass", None)
    if get is None:
        factory = message_factory.MessageFactory(pool)
        get = factory.GetPrototype
    return {n: get(pool.FindMessageTypeByName("ps." + n)) for n in ("PBNode", "PBControl", "PBMeta")}


def pack_like_van(cls, h, with_data_size=False):
    """Van::PackMeta, src/van.cc:477-514 (Van::PackMetaPB, :445-475, with_data_size)."""
    pb = cls["PBMeta"]()
    pb.head = h["head"]
    if h.get("app_id") is not None:
        pb.app_id = h["app_id"]
    if h.get("timestamp") is not None:
        pb.timestamp = h["timestamp"]
    if h.get("body"):
        pb.body = h["body"]
    pb.push = bool(h.get("push"))
    if not with_data_size:  # Van::PackMetaPB (van.cc:445-475) never calls set_pull
        pb.pull = bool(h.get("pull"))
    pb.request, pb.simple_app = bool(h.get("request")), bool(h.get("simple_app"))
    pb.priority, pb.customer_id = h.get("priority", 0), h.get("customer_id", 0)
    pb.data_type.extend(h.get("data_type", []))
    c = h.get("control")
    if c is not None and c["cmd"] != 0:
        pb.control.cmd = c["cmd"]
        if c["cmd"] == BARRIER:
            pb.control.barrier_group = c.get("barrier_group", 0)
        elif c["cmd"] == ACK:
            pb.control.msg_sig = c.get("msg_sig", 0)
        for n in c.get("nodes", []):
            p = pb.control.node.add()
            p.id = EMPTY if n.get("id") is None else n["id"]
            p.role, p.port = n["role"], n.get("port", 0)
            p.hostname = n.get("hostname", b"").decode("latin-1")
            p.is_recovery, p.customer_id = bool(n.get("is_recovery")), n.get("customer_id", 0)
    if with_data_size:
        pb.data_size = h.get("data_size", 0)
    return pb.SerializeToString()


def cases():
    node = lambda **k: dict({"role": 0, "id": None, "port": 0, "customer_id": 0, "is_recovery": False,
                             "hostname": b""}, **k)
    base = {"head": EMPTY, "app_id": None, "customer_id": EMPTY, "timestamp": None, "request": False,
            "push": False, "pull": False, "simple_app": False, "body": b"", "data_type": [], "control": None,
            "data_size": 0, "priority": 0}
    out = [("default-constructed Meta (message.h:118-121)", dict(base))]
    # a KVWorker push of keys + float values (kv_app.h:590-612): request, push, app 0, customer 0
    out.append(("kv push request", dict(base, head=0, app_id=0, customer_id=0, timestamp=7, request=True,
                                        push=True, data_type=[8, 9], data_size=12000)))
    out.append(("kv pull response with lens", dict(base, head=0, app_id=3, customer_id=1, timestamp=123456,
                                                   pull=True, data_type=[8, 9, 3], priority=2)))
    out.append(("simple app with body", dict(base, head=-5, app_id=1, customer_id=0, timestamp=0,
                                             request=True, simple_app=True, body=b"hello \x00\xff body")))
    out.append(("negative numbers take ten bytes", dict(base, head=-1, app_id=-2147483648, customer_id=-3,
                                                        timestamp=-4, priority=-1, data_type=[-1, 0, 300])))
    out.append(("barrier", dict(base, head=0, customer_id=0, request=True,
                                control={"cmd": 3, "barrier_group": 7, "msg_sig": 0, "nodes": []})))
    out.append(("ack with a 64-bit signature", dict(base, head=0, customer_id=0,
                                                    control={"cmd": 4, "barrier_group": 0,
                                                             "msg_sig": 0xFEDCBA9876543210, "nodes": []})))
    out.append(("add_node with three nodes", dict(base, head=0, customer_id=0, request=True, control={
        "cmd": 2, "barrier_group": 0, "msg_sig": 0,
        "nodes": [node(role=2, id=1, port=8000, hostname=b"127.0.0.1"),
                  node(role=0, id=None, port=53412, hostname=b"node-17.cluster.example", customer_id=4),
                  node(role=1, id=9, port=1, hostname=b"", is_recovery=True)]})))
    out.append(("heartbeat", dict(base, head=0, customer_id=0, timestamp=99,
                                  control={"cmd": 5, "barrier_group": 0, "msg_sig": 0,
                                           "nodes": [node(role=1, id=11, port=9000, hostname=b"w")]})))
    out.append(("terminate", dict(base, head=0, customer_id=0,
                                  control={"cmd": 1, "barrier_group": 0, "msg_sig": 0, "nodes": []})))
    out.append(("large body and many types", dict(base, head=1, app_id=2, customer_id=3, timestamp=4,
                                                  body=bytes(range(256)) * 3, data_type=list(range(12)) * 20)))
    return out


def jsonable(h):
    def enc(v):
        if isinstance(v, bytes):
            return {"hex": v.hex()}
        if isinstance(v, dict):
            return {k: enc(x) for k, x in v.items()}
        if isinstance(v, list):
            return [enc(x) for x in v]
        return v
    return enc(h)


def main():
    cls = pb_classes()
    rows = []
    for name, h in cases():
        rows.append({"name": name, "header": jsonable(h), "bytes": pack_like_van(cls, h).hex(),
                     "bytes_with_data_size": pack_like_van(cls, h, True).hex()})
    doc = {"source": "protobuf Python runtime %s serialising PBMeta as declared in src/meta.proto:8-60, "
                     "filled like Van::PackMeta (src/van.cc:477-514)" % google.protobuf.__version__,
           "cases": rows}
    with open(os.path.join(HERE, "meta_golden.json"), "w") as f:
        json.dump(doc, f, indent=1)
    print("wrote %d cases" % len(rows))


if __name__ == "__main__":
    sys.exit(main())
