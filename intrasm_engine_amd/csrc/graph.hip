// hipGraph builder: turns per-stream stream-captures into branches of ONE graph.
//
// Model (the behaviour of CUDAExperimentalGraphConstructor<cudaStream_t> and
// CudaGraphWrapper, common/include/helper_CUDAGraphConstructor.cu.h:106-166, 268-486):
//   * the graph starts with one empty root node;
//   * every registered stream remembers its "last activity" node (initially the root);
//   * begin_capture(stream) starts a capture INTO the graph that depends on that node,
//     end_capture(stream) ends it and moves the stream's last activity to the tail of
//     what was captured; two streams captured one after the other therefore become two
//     independent branches under the root;
//   * join adds an empty node that depends on the last activity of several streams;
//   * explicit event-record / event-wait nodes can be chained on a stream.
// Differences from the reference, on purpose: the tail of a capture is found from the set
// of nodes the capture added (several leaves are tied by an empty node) instead of walking
// a chain, so captures that fork internally are handled; join also depends on the
// destination stream's own tail.
#include "iex_common.h"

#include <algorithm>
#include <map>
#include <set>
#include <vector>

struct iex_graph {
  hipGraph_t graph = nullptr;
  hipGraphNode_t root = nullptr;
  hipGraphExec_t exec = nullptr;
  bool owns_graph = true;
  std::map<hipStream_t, hipGraphNode_t> last;  // stream -> last activity
  std::set<hipGraphNode_t> known;              // nodes seen before the running capture
  std::set<hipStream_t> capturing;
};

namespace {

using iex::check_hip;
using iex::fail;

int get_nodes(hipGraph_t g, std::vector<hipGraphNode_t>& nodes) {
  size_t n = 0;
  if (int rc = check_hip(hipGraphGetNodes(g, nullptr, &n), "hipGraphGetNodes")) return rc;
  nodes.resize(n);
  if (n == 0) return 0;
  if (int rc = check_hip(hipGraphGetNodes(g, nodes.data(), &n), "hipGraphGetNodes")) return rc;
  nodes.resize(n);
  return 0;
}

int get_edges(hipGraph_t g, std::vector<hipGraphNode_t>& from, std::vector<hipGraphNode_t>& to) {
  size_t n = 0;
  if (int rc = check_hip(hipGraphGetEdges(g, nullptr, nullptr, &n), "hipGraphGetEdges")) return rc;
  from.resize(n);
  to.resize(n);
  if (n == 0) return 0;
  if (int rc = check_hip(hipGraphGetEdges(g, from.data(), to.data(), &n), "hipGraphGetEdges")) return rc;
  from.resize(n);
  to.resize(n);
  return 0;
}

int refresh_known(iex_graph* g) {
  std::vector<hipGraphNode_t> nodes;
  if (int rc = get_nodes(g->graph, nodes)) return rc;
  g->known.insert(nodes.begin(), nodes.end());
  return 0;
}

}  // namespace

extern "C" {

iex_graph* iex_graph_create(void) {
  iex_graph* g = new iex_graph();
  if (check_hip(hipGraphCreate(&g->graph, 0), "hipGraphCreate") ||
      check_hip(hipGraphAddEmptyNode(&g->root, g->graph, nullptr, 0), "hipGraphAddEmptyNode(root)")) {
    if (g->graph) (void)hipGraphDestroy(g->graph);
    delete g;
    return nullptr;
  }
  g->known.insert(g->root);
  return g;
}

iex_graph* iex_graph_wrap(void* hip_graph) {
  if (!hip_graph) {
    fail(IEX_ERR_BAD_ARGUMENT, "graph_wrap: null graph handle");
    return nullptr;
  }
  iex_graph* g = new iex_graph();
  g->graph = static_cast<hipGraph_t>(hip_graph);
  g->owns_graph = true;  // the wrapper takes ownership, like CudaGraphWrapper(cudaGraph_t)
  (void)refresh_known(g);
  return g;
}

void iex_graph_destroy(iex_graph* g) {
  if (!g) return;
  if (g->exec) (void)hipGraphExecDestroy(g->exec);
  if (g->graph && g->owns_graph) (void)hipGraphDestroy(g->graph);
  delete g;
}

void* iex_graph_handle(iex_graph* g) { return g ? g->graph : nullptr; }

int iex_graph_register_stream(iex_graph* g, void* stream) {
  IEX_REQUIRE(g, IEX_ERR_BAD_ARGUMENT, "graph: null builder");
  IEX_REQUIRE(g->root, IEX_ERR_STATE, "graph: a wrapped graph has no root to register streams on");
  g->last[static_cast<hipStream_t>(stream)] = g->root;
  return 0;
}

int iex_graph_begin_capture(iex_graph* g, void* stream) {
  IEX_REQUIRE(g, IEX_ERR_BAD_ARGUMENT, "graph: null builder");
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto it = g->last.find(s);
  IEX_REQUIRE(it != g->last.end(), IEX_ERR_STATE, "graph: stream %p is not registered", stream);
  IEX_REQUIRE(!g->capturing.count(s), IEX_ERR_STATE, "graph: stream %p is already capturing", stream);
  IEX_REQUIRE(s != nullptr, IEX_ERR_STATE,
              "graph: captures must run on a non-default stream (it is fine to launch the graph on one)");
  IEX_REQUIRE(!g->exec, IEX_ERR_STATE, "graph: already instantiated; destroy the executable graph first");
  if (int rc = refresh_known(g)) return rc;
  hipGraphNode_t dep = it->second;
  if (int rc = check_hip(hipStreamBeginCaptureToGraph(s, g->graph, &dep, nullptr, 1, hipStreamCaptureModeGlobal),
                         "hipStreamBeginCaptureToGraph"))
    return rc;
  g->capturing.insert(s);
  return 0;
}

int iex_graph_end_capture(iex_graph* g, void* stream) {
  IEX_REQUIRE(g, IEX_ERR_BAD_ARGUMENT, "graph: null builder");
  hipStream_t s = static_cast<hipStream_t>(stream);
  IEX_REQUIRE(g->capturing.count(s), IEX_ERR_STATE, "graph: stream %p is not capturing", stream);
  g->capturing.erase(s);
  hipGraph_t out = nullptr;
  if (int rc = check_hip(hipStreamEndCapture(s, &out), "hipStreamEndCapture")) return rc;
  // Tail of the capture = the nodes it added that no other added node depends on.
  std::vector<hipGraphNode_t> nodes, from, to;
  if (int rc = get_nodes(g->graph, nodes)) return rc;
  if (int rc = get_edges(g->graph, from, to)) return rc;
  std::set<hipGraphNode_t> fresh;
  for (hipGraphNode_t n : nodes)
    if (!g->known.count(n)) fresh.insert(n);
  if (fresh.empty()) return 0;  // nothing was recorded: last activity unchanged
  std::set<hipGraphNode_t> has_fresh_successor;
  for (size_t i = 0; i < from.size(); ++i)
    if (fresh.count(from[i]) && fresh.count(to[i])) has_fresh_successor.insert(from[i]);
  std::vector<hipGraphNode_t> leaves;
  for (hipGraphNode_t n : nodes)  // node order, so the result does not depend on pointer values
    if (fresh.count(n) && !has_fresh_successor.count(n)) leaves.push_back(n);
  hipGraphNode_t tail = nullptr;
  if (leaves.size() == 1) {
    tail = leaves[0];
  } else {
    if (int rc = check_hip(hipGraphAddEmptyNode(&tail, g->graph, leaves.data(), leaves.size()),
                           "hipGraphAddEmptyNode(capture tail)"))
      return rc;
    g->known.insert(tail);
  }
  g->known.insert(fresh.begin(), fresh.end());
  g->last[s] = tail;
  return 0;
}

int iex_graph_add_event_record_node(iex_graph* g, void* event, void* stream) {
  IEX_REQUIRE(g, IEX_ERR_BAD_ARGUMENT, "graph: null builder");
  IEX_REQUIRE(event, IEX_ERR_BAD_ARGUMENT, "graph: null event (record it once so that it exists)");
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto it = g->last.find(s);
  IEX_REQUIRE(it != g->last.end(), IEX_ERR_STATE, "graph: stream %p is not registered", stream);
  hipGraphNode_t node = nullptr, dep = it->second;
  if (int rc = check_hip(hipGraphAddEventRecordNode(&node, g->graph, &dep, 1, static_cast<hipEvent_t>(event)),
                         "hipGraphAddEventRecordNode"))
    return rc;
  g->known.insert(node);
  it->second = node;
  return 0;
}

int iex_graph_add_stream_wait_event_node(iex_graph* g, void* stream, void* event) {
  IEX_REQUIRE(g, IEX_ERR_BAD_ARGUMENT, "graph: null builder");
  IEX_REQUIRE(event, IEX_ERR_BAD_ARGUMENT, "graph: null event (record it once so that it exists)");
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto it = g->last.find(s);
  IEX_REQUIRE(it != g->last.end(), IEX_ERR_STATE, "graph: stream %p is not registered", stream);
  hipGraphNode_t node = nullptr, dep = it->second;
  if (int rc = check_hip(hipGraphAddEventWaitNode(&node, g->graph, &dep, 1, static_cast<hipEvent_t>(event)),
                         "hipGraphAddEventWaitNode"))
    return rc;
  g->known.insert(node);
  it->second = node;
  return 0;
}

int iex_graph_join(iex_graph* g, void* const* streams, int num_streams, void* dst_stream) {
  IEX_REQUIRE(g, IEX_ERR_BAD_ARGUMENT, "graph: null builder");
  IEX_REQUIRE(num_streams >= 0 && (num_streams == 0 || streams), IEX_ERR_BAD_ARGUMENT, "graph: bad stream list");
  hipStream_t dst = static_cast<hipStream_t>(dst_stream);
  IEX_REQUIRE(g->last.count(dst), IEX_ERR_STATE, "graph: destination stream %p is not registered", dst_stream);
  std::vector<hipGraphNode_t> deps;
  auto add = [&](hipGraphNode_t n) {
    if (std::find(deps.begin(), deps.end(), n) == deps.end()) deps.push_back(n);
  };
  for (int i = 0; i < num_streams; ++i) {
    auto it = g->last.find(static_cast<hipStream_t>(streams[i]));
    IEX_REQUIRE(it != g->last.end(), IEX_ERR_STATE, "graph: stream %p is not registered", streams[i]);
    add(it->second);
  }
  add(g->last[dst]);
  hipGraphNode_t node = nullptr;
  if (int rc = check_hip(hipGraphAddEmptyNode(&node, g->graph, deps.data(), deps.size()), "hipGraphAddEmptyNode(join)"))
    return rc;
  g->known.insert(node);
  g->last[dst] = node;
  return 0;
}

int iex_graph_instantiate(iex_graph* g) {
  IEX_REQUIRE(g, IEX_ERR_BAD_ARGUMENT, "graph: null builder");
  IEX_REQUIRE(!g->exec, IEX_ERR_STATE, "graph: executable graph already instantiated");
  IEX_REQUIRE(g->capturing.empty(), IEX_ERR_STATE, "graph: a capture is still open");
  return check_hip(hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0), "hipGraphInstantiate");
}

int iex_graph_launch(iex_graph* g, void* stream) {
  IEX_REQUIRE(g, IEX_ERR_BAD_ARGUMENT, "graph: null builder");
  IEX_REQUIRE(g->exec, IEX_ERR_STATE, "graph: not instantiated");
  return check_hip(hipGraphLaunch(g->exec, static_cast<hipStream_t>(stream)), "hipGraphLaunch");
}

int iex_graph_destroy_exec(iex_graph* g) {
  IEX_REQUIRE(g, IEX_ERR_BAD_ARGUMENT, "graph: null builder");
  if (!g->exec) return 0;
  hipGraphExec_t e = g->exec;
  g->exec = nullptr;
  return check_hip(hipGraphExecDestroy(e), "hipGraphExecDestroy");
}

int iex_graph_add_child_graph(iex_graph* parent, iex_graph* child) {
  IEX_REQUIRE(parent && child, IEX_ERR_BAD_ARGUMENT, "graph: null builder");
  IEX_REQUIRE(!parent->exec, IEX_ERR_STATE, "graph: parent already instantiated");
  hipGraphNode_t node = nullptr;
  // The child graph is cloned into the node, so both objects stay independently owned.
  int rc = check_hip(hipGraphAddChildGraphNode(&node, parent->graph, parent->root ? &parent->root : nullptr,
                                               parent->root ? 1 : 0, child->graph),
                     "hipGraphAddChildGraphNode");
  if (rc) return rc;
  parent->known.insert(node);
  return 0;
}

iex_graph* iex_graph_combine(iex_graph* const* graphs, int num_graphs) {
  if (!graphs || num_graphs <= 0) {
    fail(IEX_ERR_BAD_ARGUMENT, "graph_combine: empty list");
    return nullptr;
  }
  iex_graph* g = new iex_graph();
  if (check_hip(hipGraphCreate(&g->graph, 0), "hipGraphCreate")) {
    delete g;
    return nullptr;
  }
  for (int i = 0; i < num_graphs; ++i) {
    hipGraphNode_t node = nullptr;
    if (!graphs[i] || check_hip(hipGraphAddChildGraphNode(&node, g->graph, nullptr, 0, graphs[i]->graph),
                                "hipGraphAddChildGraphNode(sibling)")) {
      iex_graph_destroy(g);
      return nullptr;
    }
    g->known.insert(node);
  }
  return g;
}

int iex_graph_dump_dot(iex_graph* g, const char* path) {
  IEX_REQUIRE(g && path, IEX_ERR_BAD_ARGUMENT, "graph: null argument");
  return check_hip(hipGraphDebugDotPrint(g->graph, path, hipGraphDebugDotFlagsVerbose), "hipGraphDebugDotPrint");
}

long long iex_graph_num_nodes(iex_graph* g) {
  if (!g) return IEX_ERR_BAD_ARGUMENT;
  std::vector<hipGraphNode_t> nodes;
  if (get_nodes(g->graph, nodes)) return -1;
  return (long long)nodes.size();
}

long long iex_graph_num_edges(iex_graph* g) {
  if (!g) return IEX_ERR_BAD_ARGUMENT;
  std::vector<hipGraphNode_t> from, to;
  if (get_edges(g->graph, from, to)) return -1;
  return (long long)from.size();
}

long long iex_graph_get_edges(iex_graph* g, long long* from_idx, long long* to_idx, long long cap) {
  if (!g) return IEX_ERR_BAD_ARGUMENT;
  std::vector<hipGraphNode_t> nodes, from, to;
  if (get_nodes(g->graph, nodes) || get_edges(g->graph, from, to)) return -1;
  std::map<hipGraphNode_t, long long> index;
  for (size_t i = 0; i < nodes.size(); ++i) index[nodes[i]] = (long long)i;
  for (size_t i = 0; i < from.size() && (long long)i < cap; ++i) {
    from_idx[i] = index.count(from[i]) ? index[from[i]] : -1;
    to_idx[i] = index.count(to[i]) ? index[to[i]] : -1;
  }
  return (long long)from.size();
}

int iex_graph_node_type(iex_graph* g, long long idx) {
  if (!g) return IEX_ERR_BAD_ARGUMENT;
  std::vector<hipGraphNode_t> nodes;
  if (get_nodes(g->graph, nodes)) return -1;
  if (idx < 0 || idx >= (long long)nodes.size()) return fail(IEX_ERR_BAD_ARGUMENT, "graph: node index out of range");
  hipGraphNodeType t;
  if (check_hip(hipGraphNodeGetType(nodes[idx], &t), "hipGraphNodeGetType")) return -1;
  return (int)t;
}

int iex_stream_is_capturing(void* stream) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(static_cast<hipStream_t>(stream), &st) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return st == hipStreamCaptureStatusActive ? 1 : 0;
}

}  // extern "C"
