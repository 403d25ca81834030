// pskv::PackMeta / pskv::UnpackMeta (include/pskv/meta_codec.h) on ps::Meta.
// With -DWITH_REAL_PSLITE the file only has to compile: the templates are instantiated with
// the reference's own ps::Meta (include/ps/internal/message.h). Without it, a mirror of that
// struct makes a program that packs, unpacks and compares.
#include <chrono>
#include <climits>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#ifdef WITH_REAL_PSLITE
#include "ps/internal/message.h"
#else
namespace ps {
enum DataType { CHAR, INT8, INT16, INT32, INT64, UINT8, UINT16, UINT32, UINT64, FLOAT, DOUBLE, OTHER };
struct Node {
  enum Role { SERVER, WORKER, SCHEDULER };
  Node() : id(INT_MAX), port(INT_MAX), is_recovery(false) {}
  Role role;
  int id;
  int customer_id;
  std::string hostname;
  int port;
  bool is_recovery;
};
struct Control {
  enum Command { EMPTY, TERMINATE, ADD_NODE, BARRIER, ACK, HEARTBEAT };
  Control() : cmd(EMPTY) {}
  Command cmd;
  std::vector<Node> node;
  int barrier_group;
  uint64_t msg_sig;
};
struct Meta {
  Meta() : head(INT_MAX), app_id(INT_MAX), customer_id(INT_MAX), timestamp(INT_MAX), sender(INT_MAX),
           recver(INT_MAX), request(false), push(false), pull(false), simple_app(false) {}
  int head, app_id, customer_id, timestamp, sender, recver;
  bool request, push, pull, simple_app;
  std::string body;
  std::vector<DataType> data_type;
  Control control;
  int data_size = 0;
  int priority = 0;
};
}  // namespace ps
#endif

#include "pskv/meta_codec.h"

// instantiate both templates with ps::Meta
template void pskv::PackMeta<ps::Meta>(const ps::Meta&, char**, int*);
template bool pskv::UnpackMeta<ps::Meta>(const char*, int, ps::Meta*);

#ifndef WITH_REAL_PSLITE
int main() {
  ps::Meta m;
  m.head = 3;
  m.app_id = 0;
  m.customer_id = 1;
  m.timestamp = 42;
  m.request = true;
  m.push = true;
  m.body = std::string("b\0dy", 4);
  m.data_type = {ps::UINT64, ps::FLOAT, ps::INT32};
  m.priority = -7;
  m.control.cmd = ps::Control::ADD_NODE;
  ps::Node n;
  n.role = ps::Node::WORKER;
  n.id = 9;
  n.customer_id = 2;
  n.hostname = "10.0.0.1";
  n.port = 8123;
  n.is_recovery = true;
  m.control.node.push_back(n);
  n.id = INT_MAX;  // unset
  n.hostname = "";
  m.control.node.push_back(n);
  char* buf = nullptr;
  int size = 0;
  pskv::PackMeta(m, &buf, &size);
  ps::Meta u;
  bool ok = pskv::UnpackMeta(buf, size, &u);
  ok = ok && u.head == 3 && u.app_id == 0 && u.customer_id == 1 && u.timestamp == 42 && u.request && u.push &&
       !u.pull && !u.simple_app && u.body == m.body && u.data_type == m.data_type && u.priority == -7 &&
       u.control.cmd == ps::Control::ADD_NODE && u.control.node.size() == 2 &&
       u.control.node[0].role == ps::Node::WORKER && u.control.node[0].id == 9 &&
       u.control.node[0].hostname == "10.0.0.1" && u.control.node[0].port == 8123 &&
       u.control.node[0].is_recovery && u.control.node[0].customer_id == 2 &&
       u.control.node[1].id == INT_MAX && u.control.node[1].hostname.empty();
  ok = ok && !pskv::UnpackMeta(buf, size - 1, &u);  // a cut buffer is refused
  ps::Meta plain;                                   // no control block: cmd reads EMPTY (van.cc:554-556)
  plain.head = 0;
  plain.customer_id = 0;
  delete[] buf;
  pskv::PackMeta(plain, &buf, &size);
  ps::Meta v;
  v.control.cmd = ps::Control::BARRIER;
  ok = ok && pskv::UnpackMeta(buf, size, &v) && v.control.cmd == ps::Control::EMPTY && v.app_id == INT_MAX &&
       v.timestamp == INT_MAX;
  delete[] buf;
  // the header of a KVWorker push (kv_app.h:590-612), packed and unpacked in a loop
  ps::Meta kv;
  kv.head = 0;
  kv.app_id = 0;
  kv.customer_id = 0;
  kv.timestamp = 1234;
  kv.request = kv.push = true;
  kv.data_type = {ps::UINT64, ps::FLOAT};
  const int reps = 200000;
  size_t bytes = 0;
  const auto t0 = std::chrono::steady_clock::now();
  for (int i = 0; i < reps; ++i) {
    kv.timestamp = i;
    pskv::PackMeta(kv, &buf, &size);
    ps::Meta back;
    ok = ok && pskv::UnpackMeta(buf, size, &back) && back.timestamp == i;
    bytes += size;
    delete[] buf;
  }
  const double ns = std::chrono::duration<double, std::nano>(std::chrono::steady_clock::now() - t0).count();
  std::printf("kv push header: %.1f bytes, pack + unpack %.0f ns per message\n", (double)bytes / reps, ns / reps);
  std::printf(ok ? "meta_codec_check: ok\n" : "meta_codec_check: FAILED\n");
  return ok ? 0 : 1;
}
#endif
