// HIP graph capture and replay of a step's kernel launches.
//
// The reference captures the layers of a decode-only step in a CUDA graph per batch-size
// bucket and replays it with the step's values copied into static buffers
// (src/model/paged_decoder.py:385-507).  Here the step's launches are recorded from the
// engine's own stream between ps_graph_begin and ps_graph_end; all per-step values live in
// one device buffer that is refreshed by a copy before each replay, so nothing inside the
// graph changes from step to step.  No memset node is ever recorded (buffers are cleared by
// kernels).
#include "common.h"
#include "pagedserve_hip.h"

extern "C" int ps_graph_begin(void* stream) {
  hipError_t status = hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal);
  PS_REQUIRE(status == hipSuccess, "ps_graph_begin: %s", hipGetErrorString(status));
  return 0;
}

// Ends the capture; on success *exec_out is an executable graph.
extern "C" int ps_graph_end(void* stream, void** exec_out, int* node_count) {
  hipGraph_t graph = nullptr;
  hipError_t status = hipStreamEndCapture((hipStream_t)stream, &graph);
  PS_REQUIRE(status == hipSuccess && graph != nullptr, "ps_graph_end: capture failed: %s",
             hipGetErrorString(status));
  size_t nodes = 0;
  hipGraphGetNodes(graph, nullptr, &nodes);
  if (node_count) *node_count = (int)nodes;
  hipGraphExec_t exec = nullptr;
  status = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  hipGraphDestroy(graph);
  PS_REQUIRE(status == hipSuccess && exec != nullptr, "ps_graph_end: instantiate failed: %s",
             hipGetErrorString(status));
  *exec_out = (void*)exec;
  return 0;
}

// Abandons a capture after an error inside it.
extern "C" int ps_graph_abort(void* stream) {
  hipGraph_t graph = nullptr;
  hipStreamEndCapture((hipStream_t)stream, &graph);
  if (graph) hipGraphDestroy(graph);
  (void)hipGetLastError();
  return 0;
}

extern "C" int ps_graph_launch(void* exec, void* stream) {
  hipError_t status = hipGraphLaunch((hipGraphExec_t)exec, (hipStream_t)stream);
  PS_REQUIRE(status == hipSuccess, "ps_graph_launch: %s", hipGetErrorString(status));
  return 0;
}

extern "C" int ps_graph_destroy(void* exec) {
  if (exec) hipGraphExecDestroy((hipGraphExec_t)exec);
  return 0;
}
