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

// ---- the step's metadata, fetched by a kernel ------------------------------------------------------------
// A step's token ids, positions, block tables and so on are packed on the host into pinned memory and must
// be on the device before the step's first kernel reads them. A memory copy for that goes through the copy
// engine: the compute queue hands over to it and takes over again, which on this device leaves the queue idle
// for 30 to 130 us around a copy of a few kilobytes. A kernel that reads the pinned memory itself stays in the
// step's own queue: the same bytes arrive in a few microseconds with nothing to wait for on either side.
#define TW_UPLOAD_MAX_SEGMENTS 16
struct UploadSegments {
  int n;
  int offset[TW_UPLOAD_MAX_SEGMENTS];      // in 32-bit words, the same in source and destination
  int count[TW_UPLOAD_MAX_SEGMENTS];
};

__global__ __launch_bounds__(256) void upload_words_kernel(const int* __restrict__ src, int* __restrict__ dst, UploadSegments seg) {
  for (int s = blockIdx.y; s < seg.n; s += gridDim.y) {
    const int* from = src + seg.offset[s];
    int* to = dst + seg.offset[s];
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < seg.count[s]; i += gridDim.x * blockDim.x) to[i] = from[i];
  }
}

// dst[offset[s] + i] = src[offset[s] + i] for i < count[s], s < n. `src` is pinned host memory (or any memory
// the device can read), `dst` device memory; both hold 32-bit words.
extern "C" int tw_upload_words(const int* src, int* dst, int n, const int* offsets, const int* counts, hipStream_t stream) {
  TW_REQUIRE(src != nullptr && dst != nullptr && n >= 0 && n <= TW_UPLOAD_MAX_SEGMENTS);
  if (n == 0) return 0;
  UploadSegments seg;
  seg.n = n;
  int most = 0;
  for (int s = 0; s < n; ++s) {
    TW_REQUIRE(offsets[s] >= 0 && counts[s] >= 0);
    seg.offset[s] = offsets[s];
    seg.count[s] = counts[s];
    if (counts[s] > most) most = counts[s];
  }
  int blocks = tw_div_up(most, 256);
  if (blocks > 64) blocks = 64;
  if (blocks < 1) blocks = 1;
  upload_words_kernel<<<dim3(blocks, n), 256, 0, stream>>>(src, dst, seg);
  return TW_LAUNCH_RESULT();
}

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
