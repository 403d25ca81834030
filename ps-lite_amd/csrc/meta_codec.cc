// Hand-written proto2 wire codec of ps-lite's message header: the bytes of PBMeta
// (src/meta.proto:8-60) as Van::PackMeta / Van::UnpackMeta (src/van.cc:477-557) produce
// and accept them through the protobuf runtime. Host code only.
#include <cstring>

#include "pskv/capi.h"
#include "pskv/meta_codec.h"

namespace {

// ---- writing ---------------------------------------------------------------------
// A sink that counts always and stores while there is room, so one pass gives ByteSize
// and, with a large enough buffer, the bytes.
struct Sink {
  char* buf;
  size_t cap;
  size_t at;
  void byte(uint8_t b) {
    if (buf && at < cap) buf[at] = static_cast<char>(b);
    ++at;
  }
  void varint(uint64_t v) {
    while (v >= 0x80) {
      byte(static_cast<uint8_t>(v) | 0x80);
      v >>= 7;
    }
    byte(static_cast<uint8_t>(v));
  }
  void tag(unsigned field, unsigned wire) { varint((static_cast<uint64_t>(field) << 3) | wire); }
  // int32 fields are sign-extended to 64 bits first: a negative value takes ten bytes
  void int32_field(unsigned field, int32_t v) {
    tag(field, 0);
    varint(static_cast<uint64_t>(static_cast<int64_t>(v)));
  }
  void bool_field(unsigned field, int32_t v) {
    tag(field, 0);
    byte(v ? 1 : 0);
  }
  void bytes_field(unsigned field, const char* p, size_t n) {
    tag(field, 2);
    varint(n);
    for (size_t i = 0; i < n; ++i) byte(static_cast<uint8_t>(p[i]));
  }
};

size_t varint_size(uint64_t v) {
  size_t n = 1;
  while (v >= 0x80) {
    v >>= 7;
    ++n;
  }
  return n;
}

// PBNode, meta.proto:8-21; every field is set by van.cc:500-507
void write_node(Sink& s, const pskv_meta_node& n) {
  s.int32_field(1, n.role);
  s.int32_field(2, n.id);
  s.bytes_field(3, n.hostname, n.hostname_len);
  s.int32_field(4, n.port);
  s.bool_field(5, n.is_recovery);
  s.int32_field(10, n.customer_id);
}

// PBControl, meta.proto:24-29; van.cc:493-508
void write_control(Sink& s, const pskv_meta& m) {
  s.int32_field(1, m.control_cmd);
  for (size_t i = 0; i < m.n_nodes; ++i) {
    Sink measure{nullptr, 0, 0};
    write_node(measure, m.nodes[i]);
    s.tag(2, 2);
    s.varint(measure.at);
    write_node(s, m.nodes[i]);
  }
  if (m.control_cmd == PSKV_CTRL_BARRIER) s.int32_field(3, m.barrier_group);
  if (m.control_cmd == PSKV_CTRL_ACK) {
    s.tag(4, 0);
    s.varint(m.msg_sig);
  }
}

// PBMeta, meta.proto:32-60, in field-number order; what is set: van.cc:480-491
void write_meta(Sink& s, const pskv_meta& m, bool with_data_size) {
  s.int32_field(1, m.head);
  if (m.body_len) s.bytes_field(2, m.body, m.body_len);
  if (m.control_cmd != PSKV_CTRL_EMPTY) {
    Sink measure{nullptr, 0, 0};
    write_control(measure, m);
    s.tag(3, 2);
    s.varint(measure.at);
    write_control(s, m);
  }
  s.bool_field(4, m.request);
  s.bool_field(5, m.push);
  s.bool_field(6, m.simple_app);
  if (m.app_id != PSKV_META_EMPTY) s.int32_field(7, m.app_id);
  if (m.timestamp != PSKV_META_EMPTY) s.int32_field(8, m.timestamp);
  if (m.n_data_type) {  // repeated int32 data_type = 9 [packed=true]
    size_t payload = 0;
    for (size_t i = 0; i < m.n_data_type; ++i)
      payload += varint_size(static_cast<uint64_t>(static_cast<int64_t>(m.data_type[i])));
    s.tag(9, 2);
    s.varint(payload);
    for (size_t i = 0; i < m.n_data_type; ++i)
      s.varint(static_cast<uint64_t>(static_cast<int64_t>(m.data_type[i])));
  }
  s.int32_field(10, m.customer_id);
  if (with_data_size) {
    s.int32_field(11, m.data_size);  // Van::PackMetaPB, van.cc:445-475: data_size, and pull is NOT set
  } else {
    s.bool_field(12, m.pull);        // Van::PackMeta, van.cc:485
  }
  s.int32_field(13, m.priority);
}

// ---- reading ---------------------------------------------------------------------
struct Source {
  const uint8_t* p;
  const uint8_t* end;
  bool ok;
  bool done() const { return p >= end; }
  uint64_t varint() {
    uint64_t v = 0;
    for (int shift = 0; shift < 70; shift += 7) {
      if (p >= end) break;
      const uint8_t b = *p++;
      if (shift < 64) v |= static_cast<uint64_t>(b & 0x7f) << shift;
      if (!(b & 0x80)) return v;
    }
    ok = false;  // ran off the buffer, or more than ten bytes
    return 0;
  }
  // a length-delimited payload as a sub-source; advances past it
  Source sub() {
    const uint64_t n = varint();
    if (!ok || n > static_cast<uint64_t>(end - p)) {
      ok = false;
      return Source{p, p, false};
    }
    Source s{p, p + n, true};
    p += n;
    return s;
  }
  void skip(unsigned wire) {
    switch (wire) {
      case 0: (void)varint(); break;
      case 1: if (end - p < 8) ok = false; else p += 8; break;
      case 2: (void)sub(); break;
      case 5: if (end - p < 4) ok = false; else p += 4; break;
      default: ok = false;  // groups are not part of this schema
    }
  }
};

bool read_node(Source s, pskv_meta_node* n) {
  *n = pskv_meta_node{0, PSKV_META_EMPTY, 0, 0, 0, nullptr, 0};  // van.cc:546-551 defaults
  bool has_role = false;
  while (s.ok && !s.done()) {
    const uint64_t t = s.varint();
    if (!s.ok) break;
    const unsigned field = static_cast<unsigned>(t >> 3), wire = static_cast<unsigned>(t & 7);
    if (wire == 0 && field == 1) { n->role = static_cast<int32_t>(s.varint()); has_role = true; }
    else if (wire == 0 && field == 2) n->id = static_cast<int32_t>(s.varint());
    else if (wire == 2 && field == 3) {
      Source h = s.sub();
      n->hostname = reinterpret_cast<const char*>(h.p);
      n->hostname_len = static_cast<size_t>(h.end - h.p);
    }
    else if (wire == 0 && field == 4) n->port = static_cast<int32_t>(s.varint());
    else if (wire == 0 && field == 5) n->is_recovery = s.varint() != 0;
    else if (wire == 0 && field == 10) n->customer_id = static_cast<int32_t>(s.varint());
    else s.skip(wire);
  }
  return s.ok && has_role;  // `required int32 role`
}

struct Room {
  pskv_meta_node* nodes;
  size_t nodes_cap;
  int32_t* types;
  size_t types_cap;
};

bool read_control(Source s, pskv_meta* m, const Room& room, bool* has_cmd) {
  while (s.ok && !s.done()) {
    const uint64_t t = s.varint();
    if (!s.ok) break;
    const unsigned field = static_cast<unsigned>(t >> 3), wire = static_cast<unsigned>(t & 7);
    if (wire == 0 && field == 1) { m->control_cmd = static_cast<int32_t>(s.varint()); *has_cmd = true; }
    else if (wire == 2 && field == 2) {
      Source ns = s.sub();
      if (!s.ok) break;
      pskv_meta_node n;
      if (!read_node(ns, &n)) return false;
      if (m->n_nodes < room.nodes_cap) room.nodes[m->n_nodes] = n;
      ++m->n_nodes;
    }
    else if (wire == 0 && field == 3) m->barrier_group = static_cast<int32_t>(s.varint());
    else if (wire == 0 && field == 4) m->msg_sig = s.varint();
    else s.skip(wire);
  }
  return s.ok;
}

void add_type(pskv_meta* m, const Room& room, int32_t v) {
  if (m->n_data_type < room.types_cap) room.types[m->n_data_type] = v;
  ++m->n_data_type;
}

}  // namespace

extern "C" {

int pskv_meta_pack(const pskv_meta* m, int with_data_size, char* buf, size_t cap, size_t* size) {
  if (!m || !size) return PSKV_EINVAL;
  Sink s{buf, cap, 0};
  write_meta(s, *m, with_data_size != 0);
  *size = s.at;
  return s.at <= cap && (buf || s.at == 0) ? PSKV_OK : PSKV_ESIZE_MISMATCH;
}

int pskv_meta_unpack(const char* buf, size_t size, pskv_meta* m, pskv_meta_node* nodes,
                     size_t nodes_cap, int32_t* data_type, size_t data_type_cap) {
  if (!m || (size && !buf)) return PSKV_EINVAL;
  std::memset(m, 0, sizeof(*m));
  m->app_id = PSKV_META_EMPTY;     // van.cc:524-525: kEmpty unless the field is present
  m->timestamp = PSKV_META_EMPTY;
  m->nodes = nodes;
  m->data_type = data_type;
  const Room room{nodes, nodes ? nodes_cap : 0, data_type, data_type ? data_type_cap : 0};
  const uint8_t* b = reinterpret_cast<const uint8_t*>(buf);
  Source s{b, b + size, true};
  bool has_cmd = false;
  while (s.ok && !s.done()) {
    const uint64_t t = s.varint();
    if (!s.ok) break;
    const unsigned field = static_cast<unsigned>(t >> 3), wire = static_cast<unsigned>(t & 7);
    if (field == 0) { s.ok = false; break; }
    if (wire == 0 && field == 1) m->head = static_cast<int32_t>(s.varint());
    else if (wire == 2 && field == 2) {
      Source bs = s.sub();
      m->body = reinterpret_cast<const char*>(bs.p);
      m->body_len = static_cast<size_t>(bs.end - bs.p);
    }
    else if (wire == 2 && field == 3) {
      Source cs = s.sub();
      if (!s.ok) break;
      m->has_control = 1;
      if (!read_control(cs, m, room, &has_cmd)) return PSKV_EINVAL;
    }
    else if (wire == 0 && field == 4) m->request = s.varint() != 0;
    else if (wire == 0 && field == 5) m->push = s.varint() != 0;
    else if (wire == 0 && field == 6) m->simple_app = s.varint() != 0;
    else if (wire == 0 && field == 7) m->app_id = static_cast<int32_t>(s.varint());
    else if (wire == 0 && field == 8) m->timestamp = static_cast<int32_t>(s.varint());
    else if (wire == 2 && field == 9) {  // packed
      Source ps = s.sub();
      while (ps.ok && !ps.done()) {
        const int32_t v = static_cast<int32_t>(ps.varint());
        if (ps.ok) add_type(m, room, v);
      }
      if (!ps.ok) s.ok = false;
    }
    else if (wire == 0 && field == 9) add_type(m, room, static_cast<int32_t>(s.varint()));  // unpacked
    else if (wire == 0 && field == 10) m->customer_id = static_cast<int32_t>(s.varint());
    else if (wire == 0 && field == 11) m->data_size = static_cast<int32_t>(s.varint());
    else if (wire == 0 && field == 12) m->pull = s.varint() != 0;
    else if (wire == 0 && field == 13) m->priority = static_cast<int32_t>(s.varint());
    else s.skip(wire);
  }
  if (!s.ok) return PSKV_EINVAL;
  if (m->has_control && !has_cmd) return PSKV_EINVAL;  // `required int32 cmd`
  if (m->n_nodes > room.nodes_cap || m->n_data_type > room.types_cap) return PSKV_ESIZE_MISMATCH;
  return PSKV_OK;
}

}  // extern "C"
