// Small runtime helpers: error text, HIP graph capture and replay on a stream.
#include "tw_common.h"

extern "C" const char* tw_error_string(int code) {
  if (code == TW_ERR_BAD_ARGUMENT) return "a kernel launcher refused its arguments (shape, alignment or size)";
  if (code == TW_ERR_TOO_LARGE)
    return "the input is larger than this entry point's built-in scratch memory holds (tw_sample_rows_static: at most 256 rows)";
  return hipGetErrorString((hipError_t)code);
}

extern "C" int tw_abi_version() { return 1; }

// Capture everything launched on `stream` between begin and end into a graph.
// Nothing that allocates, synchronises or sets memory may run in between.
extern "C" int tw_graph_begin(hipStream_t stream) {
  return (int)hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal);
}

extern "C" int tw_graph_end(hipStream_t stream, void** exec_out) {
  hipGraph_t graph = nullptr;
  hipError_t e = hipStreamEndCapture(stream, &graph);
  if (e != hipSuccess) return (int)e;
  hipGraphExec_t exec = nullptr;
  e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (e != hipSuccess) return (int)e;
  *exec_out = (void*)exec;
  return 0;
}

extern "C" int tw_graph_launch(void* exec, hipStream_t stream) {
  return (int)hipGraphLaunch((hipGraphExec_t)exec, stream);
}

extern "C" int tw_graph_destroy(void* exec) { return (int)hipGraphExecDestroy((hipGraphExec_t)exec); }
