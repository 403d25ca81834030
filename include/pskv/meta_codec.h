/*
 * The wire format of a ps-lite message header (ps::Meta), written by hand.
 *
 * The reference turns ps::Meta into a proto2 message PBMeta (src/meta.proto:8-60) and lets
 * the protobuf runtime serialise it: Van::PackMeta / Van::UnpackMeta, src/van.cc:477-557
 * (Van::PackMetaPB, van.cc:445-475, is the same packing plus `data_size`). The two
 * functions below produce and read the very same bytes without protobuf, so the host
 * plumbing around the GPU path needs neither protoc nor libprotobuf.
 *
 * Bytes written: fields in field-number order, each field that the reference sets
 * (van.cc:480-507) is present even when it holds its default, int32 values are
 * sign-extended to 64 bits before they become varints (a negative number takes ten
 * bytes), `data_type` is one packed field, a control block and its nodes are nested
 * length-delimited messages. This is what every protobuf runtime emits for PBMeta.
 * Bytes read: fields in any order, later values override earlier ones, repeated and nested
 * fields accumulate, packed and unpacked `data_type` are both accepted, unknown fields
 * are skipped, a missing required field (PBNode.role, PBControl.cmd) or a truncated buffer
 * is an error, as it is for PBMeta::ParseFromArray.
 */
#ifndef PSKV_META_CODEC_H_
#define PSKV_META_CODEC_H_
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* std::numeric_limits<int>::max(): Meta::kEmpty and Node::kEmpty, src/customer.cc:8-9 */
#define PSKV_META_EMPTY 2147483647

/* Control::Command, include/ps/internal/message.h:101 */
#define PSKV_CTRL_EMPTY 0
#define PSKV_CTRL_TERMINATE 1
#define PSKV_CTRL_ADD_NODE 2
#define PSKV_CTRL_BARRIER 3
#define PSKV_CTRL_ACK 4
#define PSKV_CTRL_HEARTBEAT 5

/* ps::Node (message.h:60-92) */
typedef struct pskv_meta_node {
  int32_t role;
  int32_t id;          /* PSKV_META_EMPTY when unset */
  int32_t port;
  int32_t customer_id;
  int32_t is_recovery; /* 0 or 1 */
  const char* hostname;
  size_t hostname_len;
} pskv_meta_node;

/* ps::Meta with its ps::Control (message.h:96-196). sender and recver never travel
 * (van.cc:480-507 does not pack them). Strings and arrays are views: pack reads them,
 * unpack points them into the buffer it parsed (body, hostnames) or into the arrays
 * the caller passed (nodes, data_type). */
typedef struct pskv_meta {
  int32_t head;
  int32_t app_id;      /* PSKV_META_EMPTY when unset */
  int32_t customer_id;
  int32_t timestamp;   /* PSKV_META_EMPTY when unset */
  int32_t request, push, pull, simple_app; /* 0 or 1 */
  const char* body;
  size_t body_len;
  const int32_t* data_type;
  size_t n_data_type;
  int32_t control_cmd; /* pack writes a control block unless this is PSKV_CTRL_EMPTY (van.cc:492) */
  int32_t has_control; /* set by unpack: the bytes held a control block (van.cc:538) */
  int32_t barrier_group;
  uint64_t msg_sig;
  const pskv_meta_node* nodes;
  size_t n_nodes;
  int32_t data_size;
  int32_t priority;
} pskv_meta;

/* Van::PackMeta (van.cc:477-514); with_data_size != 0 packs like Van::PackMetaPB
 * (van.cc:445-475) instead: field 11 (data_size) is written and field 12 (pull) is not, as
 * that function never sets it. Writes at most cap bytes and always sets *size to the bytes needed
 * (PBMeta::ByteSize); returns 0, or -2 (PSKV_ESIZE_MISMATCH) when cap is too small. */
int pskv_meta_pack(const pskv_meta* m, int with_data_size, char* buf, size_t cap, size_t* size);

/* Van::UnpackMeta (van.cc:516-557). nodes / data_type give room for the repeated
 * fields; *m says how many were found. Returns 0, -5 (PSKV_EINVAL) for bytes that are
 * not a PBMeta (truncated, bad wire type, missing required field), -2 when the room for
 * nodes or data types is too small (m->n_nodes / m->n_data_type then hold the counts
 * needed). */
int pskv_meta_unpack(const char* buf, size_t size, pskv_meta* m, pskv_meta_node* nodes,
                     size_t nodes_cap, int32_t* data_type, size_t data_type_cap);

#ifdef __cplusplus
} /* extern "C" */

#include <string>
#include <type_traits>
#include <vector>

namespace pskv {

/* Drop-ins for the bodies of Van::PackMeta / Van::UnpackMeta, for any type shaped like
 * ps::Meta (the real one from "ps/internal/message.h" or a mirror). */
template <typename Meta>
inline void PackMeta(const Meta& meta, char** meta_buf, int* buf_size) {
  typedef typename std::remove_reference<decltype(meta.control)>::type Control;
  std::vector<pskv_meta_node> nodes(meta.control.node.size());
  for (size_t i = 0; i < nodes.size(); ++i) {
    const auto& n = meta.control.node[i];
    nodes[i] = pskv_meta_node{static_cast<int32_t>(n.role), n.id, n.port, n.customer_id,
                              n.is_recovery ? 1 : 0, n.hostname.data(), n.hostname.size()};
  }
  std::vector<int32_t> types(meta.data_type.size());
  for (size_t i = 0; i < types.size(); ++i) types[i] = static_cast<int32_t>(meta.data_type[i]);
  pskv_meta m = pskv_meta();
  m.head = meta.head;
  m.app_id = meta.app_id;
  m.customer_id = meta.customer_id;
  m.timestamp = meta.timestamp;
  m.request = meta.request;
  m.push = meta.push;
  m.pull = meta.pull;
  m.simple_app = meta.simple_app;
  m.body = meta.body.data();
  m.body_len = meta.body.size();
  m.data_type = types.data();
  m.n_data_type = types.size();
  m.control_cmd = static_cast<int32_t>(meta.control.cmd);
  m.barrier_group = meta.control.cmd == Control::BARRIER ? meta.control.barrier_group : 0;
  m.msg_sig = meta.control.cmd == Control::ACK ? meta.control.msg_sig : 0;
  m.nodes = nodes.data();
  m.n_nodes = nodes.size();
  m.data_size = meta.data_size;
  m.priority = meta.priority;
  size_t need = 0;
  pskv_meta_pack(&m, 0, nullptr, 0, &need);
  *meta_buf = new char[need + 1];  // van.cc:511
  *buf_size = static_cast<int>(need);
  pskv_meta_pack(&m, 0, *meta_buf, need, &need);
}

/* Returns false where the reference's CHECK on ParseFromArray would fail (van.cc:519). */
template <typename Meta>
inline bool UnpackMeta(const char* meta_buf, int buf_size, Meta* meta) {
  typedef typename std::remove_reference<decltype(meta->control)>::type Control;
  typedef typename std::remove_reference<decltype(meta->control.node[0])>::type Node;
  typedef typename std::remove_reference<decltype(meta->data_type[0])>::type DataType;
  pskv_meta m;
  std::vector<pskv_meta_node> nodes(8);
  std::vector<int32_t> types(8);
  int rc = pskv_meta_unpack(meta_buf, static_cast<size_t>(buf_size), &m, nodes.data(), nodes.size(),
                            types.data(), types.size());
  if (rc == -2) {
    nodes.resize(m.n_nodes + 1);
    types.resize(m.n_data_type + 1);
    rc = pskv_meta_unpack(meta_buf, static_cast<size_t>(buf_size), &m, nodes.data(), nodes.size(),
                          types.data(), types.size());
  }
  if (rc != 0) return false;
  meta->head = m.head;
  meta->app_id = m.app_id;
  meta->timestamp = m.timestamp;
  meta->request = m.request != 0;
  meta->push = m.push != 0;
  meta->pull = m.pull != 0;
  meta->simple_app = m.simple_app != 0;
  meta->priority = m.priority;
  meta->body.assign(m.body ? m.body : "", m.body_len);
  meta->customer_id = m.customer_id;
  meta->data_type.resize(m.n_data_type);
  for (size_t i = 0; i < m.n_data_type; ++i) meta->data_type[i] = static_cast<DataType>(types[i]);
  meta->control.cmd = static_cast<decltype(meta->control.cmd)>(m.has_control ? m.control_cmd : PSKV_CTRL_EMPTY);
  if (m.has_control) {
    meta->control.barrier_group = m.barrier_group;
    meta->control.msg_sig = m.msg_sig;
    for (size_t i = 0; i < m.n_nodes; ++i) {  // van.cc:543-552 appends
      Node n;
      n.role = static_cast<decltype(n.role)>(nodes[i].role);
      n.port = nodes[i].port;
      n.hostname.assign(nodes[i].hostname ? nodes[i].hostname : "", nodes[i].hostname_len);
      n.id = nodes[i].id;
      n.is_recovery = nodes[i].is_recovery != 0;
      n.customer_id = nodes[i].customer_id;
      meta->control.node.push_back(n);
    }
  }
  (void)sizeof(Control);
  return true;
}

}  // namespace pskv
#endif /* __cplusplus */
#endif /* PSKV_META_CODEC_H_ */
