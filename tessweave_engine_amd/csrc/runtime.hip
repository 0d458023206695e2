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

// ---- a yardstick, not part of any model: how fast can this device read memory at all? --------------------
// Every wave streams 1 KB non-temporal loads, eight in flight, and adds them up; nothing is written unless
// the sum takes one particular value (so the loads cannot be dropped). Benchmarks time it over gigabytes to
// put a measured ceiling beside the nominal one.
template <int U>
__global__ __launch_bounds__(256) void probe_read_kernel(const f32x4* __restrict__ src, float* out, size_t vec_per_block) {
  const f32x4* p = src + (size_t)blockIdx.x * vec_per_block + threadIdx.x;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (size_t i = 0; i < vec_per_block; i += 256 * U) {
    f32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(p + i + u * 256);
#pragma unroll
    for (int u = 0; u < U; ++u) acc += v[u];
  }
  if (acc[0] + acc[1] + acc[2] + acc[3] == 12345.678f) out[0] = 1.f;
}

// Reads the first `blocks * floor(bytes / blocks / 32 KiB) * 32 KiB` bytes of src; returns that count in *read_bytes.
extern "C" int tw_probe_read(const void* src, long bytes, float* out, int blocks, long* read_bytes, hipStream_t stream) {
  TW_REQUIRE(src != nullptr && out != nullptr && blocks > 0 && (uintptr_t)src % 16 == 0);
  const size_t per_block = (size_t)bytes / blocks / (256 * 8 * 16) * (256 * 8);      // in 16-byte vectors
  TW_REQUIRE(per_block > 0);
  if (read_bytes) *read_bytes = (long)(per_block * 16 * blocks);
  probe_read_kernel<8><<<blocks, 256, 0, stream>>>((const f32x4*)src, out, per_block);
  return TW_LAUNCH_RESULT();
}
