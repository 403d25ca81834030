"""The hand-written wire codec of the message header against the protobuf runtime.

Golden bytes (tests/golden/meta_golden.json) were produced by the protobuf Python runtime from
PBMeta as src/meta.proto:8-60 declares it, filled the way Van::PackMeta fills it
(src/van.cc:477-514). Where that runtime can be imported the same comparison also runs live,
on random headers and on byte strings only a protobuf writer other than ps-lite would
produce (fields out of order, unset optional fields, unpacked repeated fields, unknown fields)."""
import json
import os
import subprocess

import numpy as np
import pytest

from conftest import REPO

GOLDEN = os.path.join(REPO, "tests", "golden", "meta_golden.json")
REFERENCE = "/root/reference"


@pytest.fixture(scope="module")
def meta():
    import __graft_entry__ as g
    return g.load_package().meta


def _decode(v):
    if isinstance(v, dict) and set(v) == {"hex"}:
        return bytes.fromhex(v["hex"])
    if isinstance(v, dict):
        return {k: _decode(x) for k, x in v.items()}
    if isinstance(v, list):
        return [_decode(x) for x in v]
    return v


def _cases():
    return [(c["name"], _decode(c["header"]), bytes.fromhex(c["bytes"]), bytes.fromhex(c["bytes_with_data_size"]))
            for c in json.load(open(GOLDEN))["cases"]]


def _as_unpacked(h, with_data_size=False):
    """What Van::UnpackMeta (van.cc:516-557) makes of a header packed by Van::PackMeta."""
    u = dict(h)
    u["data_size"] = h["data_size"] if with_data_size else 0
    if with_data_size:
        u["pull"] = False  # Van::PackMetaPB (van.cc:445-475) never sets it, so it does not travel
    c = h["control"]
    if c is not None:
        # only the field that belongs to the command travels (van.cc:494-498)
        u["control"] = dict(c, barrier_group=c["barrier_group"] if c["cmd"] == 3 else 0,
                            msg_sig=c["msg_sig"] if c["cmd"] == 4 else 0)
    return u


@pytest.mark.parametrize("name,header,want,want_ds", _cases(), ids=[c[0] for c in _cases()])
def test_golden_bytes(meta, name, header, want, want_ds):
    assert meta.pack(header) == want
    assert meta.pack(header, with_data_size=True) == want_ds
    assert meta.unpack(want) == _as_unpacked(header)
    assert meta.unpack(want_ds) == _as_unpacked(header, True)


def test_known_bytes_by_hand(meta):
    """Spelt out by hand from the encoding rules, so that the golden file is not the only witness:
    tag = field << 3 | wire type, varints little-endian base 128, int32 sign-extended to 64 bits."""
    h = {"head": 1, "app_id": 2, "customer_id": 3, "timestamp": 300, "request": True, "push": False,
         "pull": True, "simple_app": False, "body": b"ab", "data_type": [1, 128], "control": None,
         "data_size": 0, "priority": -1}
    want = bytes([0x08, 0x01,                    # 1: head = 1
                  0x12, 0x02, 0x61, 0x62,        # 2: body = "ab"
                  0x20, 0x01,                    # 4: request
                  0x28, 0x00,                    # 5: push
                  0x30, 0x00,                    # 6: simple_app
                  0x38, 0x02,                    # 7: app_id
                  0x40, 0xAC, 0x02,              # 8: timestamp = 300
                  0x4A, 0x03, 0x01, 0x80, 0x01,  # 9: packed {1, 128}
                  0x50, 0x03,                    # 10: customer_id
                  0x60, 0x01,                    # 12: pull
                  0x68] + [0xFF] * 9 + [0x01])   # 13: priority = -1, ten bytes
    assert meta.pack(h) == want
    assert meta.unpack(want) == h


def _random_header(rng):
    def i32():
        return int(rng.choice([0, 1, -1, 127, 128, 300, 2 ** 31 - 2, -2 ** 31, int(rng.integers(-2 ** 31, 2 ** 31 - 1))]))
    h = {"head": i32(), "app_id": None if rng.random() < 0.3 else i32(), "customer_id": i32(),
         "timestamp": None if rng.random() < 0.3 else i32(), "request": bool(rng.integers(2)),
         "push": bool(rng.integers(2)), "pull": bool(rng.integers(2)), "simple_app": bool(rng.integers(2)),
         "body": bytes(rng.integers(0, 256, size=int(rng.choice([0, 0, 1, 5, 200, 70000]))).astype(np.uint8)),
         "data_type": [i32() for _ in range(int(rng.choice([0, 0, 1, 2, 3, 40])))], "control": None,
         "data_size": i32(), "priority": i32()}
    if h["app_id"] == 2 ** 31 - 1:
        h["app_id"] = None
    if h["timestamp"] == 2 ** 31 - 1:
        h["timestamp"] = None
    if rng.random() < 0.5:
        cmd = int(rng.integers(1, 6))
        nodes = []
        for _ in range(int(rng.choice([0, 1, 2, 9, 20]))):
            nid = None if rng.random() < 0.3 else i32()
            nodes.append({"role": int(rng.integers(0, 3)), "id": None if nid == 2 ** 31 - 1 else nid, "port": i32(),
                          "customer_id": i32(), "is_recovery": bool(rng.integers(2)),
                          "hostname": bytes(rng.integers(32, 127, size=int(rng.integers(0, 40))).astype(np.uint8))})
        h["control"] = {"cmd": cmd, "barrier_group": i32(), "msg_sig": int(rng.integers(0, 2 ** 63)) * 2 + 1,
                        "nodes": nodes}
    return h


def _protobuf():
    try:
        import importlib.util
        spec = importlib.util.spec_from_file_location(
            "make_meta_golden", os.path.join(REPO, "tests", "golden", "make_meta_golden.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        return mod, mod.pb_classes()
    except ImportError:
        pytest.skip("the protobuf runtime is not importable here; the golden bytes cover this")


def test_random_headers_against_protobuf(meta):
    gen, cls = _protobuf()
    rng = np.random.default_rng(2024)
    for _ in range(400):
        h = _random_header(rng)
        for ds in (False, True):
            want = gen.pack_like_van(cls, h, ds)
            assert meta.pack(h, with_data_size=ds) == want
            assert meta.unpack(want) == _as_unpacked(h, ds)


def test_reads_what_other_protobuf_writers_produce(meta):
    """UnpackMeta goes through a full protobuf parser (van.cc:519), so it accepts any valid encoding."""
    gen, cls = _protobuf()
    pb = cls["PBMeta"]()
    pb.timestamp = 5  # nothing else set: every other field reads as its default
    h = meta.unpack(pb.SerializeToString())
    assert h == {"head": 0, "app_id": None, "customer_id": 0, "timestamp": 5, "request": False, "push": False,
                 "pull": False, "simple_app": False, "body": b"", "data_type": [], "data_size": 0, "priority": 0,
                 "control": None}
    # a control block without nodes whose only field is the required cmd; a node without optional fields
    pb = cls["PBMeta"]()
    pb.control.cmd = 0
    n = pb.control.node.add()
    n.role = 2
    h = meta.unpack(pb.SerializeToString())
    assert h["control"] == {"cmd": 0, "barrier_group": 0, "msg_sig": 0,
                            "nodes": [{"role": 2, "id": None, "port": 0, "customer_id": 0, "is_recovery": False,
                                       "hostname": b""}]}
    # fields out of order, a scalar twice (the last one wins), data_type unpacked and in two packed runs,
    # two control blocks (they merge), unknown fields of every wire type in between
    raw = bytes([0x68, 0x07,                          # priority = 7
                 0x48, 0x05,                          # data_type, unpacked: 5
                 0x4A, 0x02, 0x06, 0x07,              # data_type, packed: 6, 7
                 0xF8, 0x01, 0x2A,                    # unknown field 31, varint
                 0xF9, 0x01] + [0] * 8 + [            # unknown field 31, 64-bit
                 0xFA, 0x01, 0x03, 0x01, 0x02, 0x03,  # unknown field 31, length-delimited
                 0xFD, 0x01, 0x00, 0x00, 0x00, 0x00,  # unknown field 31, 32-bit
                 0x1A, 0x02, 0x08, 0x03,              # control { cmd = 3 }
                 0x08, 0x01,                          # head = 1
                 0x1A, 0x02, 0x18, 0x09,              # control { barrier_group = 9 }
                 0x08, 0x02,                          # head = 2
                 0x48, 0x08])                         # data_type: 8
    pb = cls["PBMeta"]()
    pb.ParseFromString(raw)
    assert (pb.head, pb.priority, list(pb.data_type), pb.control.cmd, pb.control.barrier_group) == (2, 7, [5, 6, 7, 8], 3, 9)
    h = meta.unpack(raw)
    assert (h["head"], h["priority"], h["data_type"]) == (2, 7, [5, 6, 7, 8])
    assert h["control"] == {"cmd": 3, "barrier_group": 9, "msg_sig": 0, "nodes": []}
    assert h["app_id"] is None and h["timestamp"] is None


def test_rejects_what_parse_from_array_rejects(meta, capi):
    good = bytes.fromhex(json.load(open(GOLDEN))["cases"][7]["bytes"])  # add_node with three nodes
    assert meta.unpack(good)["control"]["cmd"] == 2
    bad = [good[:-1],                      # cut inside the last field
           good[:10],                      # cut inside the control block
           bytes([0x08]),                  # a tag without its value
           bytes([0x08] + [0xFF] * 11),    # a varint longer than ten bytes
           bytes([0x12, 0x05, 0x61]),      # a length that reaches past the end
           bytes([0x0B]),                  # wire type 3 (group) is not part of the schema
           bytes([0x00, 0x00]),            # field number 0
           bytes([0x1A, 0x00]),            # control without its required cmd
           bytes([0x1A, 0x04, 0x08, 0x02, 0x12, 0x00])]  # a node without its required role
    for b in bad:
        with pytest.raises(capi.PskvError) as e:
            meta.unpack(b)
        assert e.value.code == capi.EINVAL, b.hex()
    try:
        gen, cls = _protobuf()
    except pytest.skip.Exception:
        return
    from google.protobuf.message import DecodeError
    for b in bad:
        with pytest.raises(DecodeError):
            pb = cls["PBMeta"]()
            pb.ParseFromString(b)
            if not pb.IsInitialized():  # the C++ lite runtime of the reference fails the parse itself
                raise DecodeError("missing required field")


def test_header_is_plain_c_and_exported(tmp_path, capi):
    src = tmp_path / "use.c"
    src.write_text('#include "pskv/meta_codec.h"\nint main(void){ pskv_meta m; size_t n; m.head = 0; '
                   '(void)m; (void)n; return PSKV_CTRL_EMPTY; }\n')
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I" + os.path.join(REPO, "include"), "-c", str(src),
                    "-o", str(tmp_path / "use.o")], check=True)
    lib = capi.load()
    assert hasattr(lib, "pskv_meta_pack") and hasattr(lib, "pskv_meta_unpack")


def test_templates_fit_the_real_message_header(tmp_path):
    """pskv::PackMeta / pskv::UnpackMeta take the reference's own ps::Meta; and, on a mirror of it, a
    round trip through both gives the header back."""
    src = os.path.join(REPO, "tests", "meta_codec_check.cc")
    inc = ["-I" + os.path.join(REPO, "include")]
    if os.path.exists(os.path.join(REFERENCE, "include", "ps", "internal", "message.h")):
        subprocess.run(["g++", "-std=c++11", "-Wall", "-DWITH_REAL_PSLITE", "-I" + os.path.join(REFERENCE, "include")]
                       + inc + ["-c", src, "-o", str(tmp_path / "real.o")], check=True)
    exe = str(tmp_path / "meta_check")
    lib = os.path.join(REPO, "ps-lite_amd")
    subprocess.run(["g++", "-std=c++11", "-Wall"] + inc + [src, "-L" + lib, "-lpskv", "-Wl,-rpath," + lib,
                    "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib", "-lamdhip64", "-o", exe], check=True)
    r = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
    assert r.returncode == 0 and "meta_codec_check: ok" in r.stdout, r.stdout
