// Next-token choice per logits row: greedy (temperature 0: the lowest index among
// the largest logits) or temperature sampling by inverse CDF over
// softmax(logits / T), all in float32. The uniform number of a row comes from a
// counter-based generator keyed by (the request's seed, the index of the token
// being drawn), so a request's stream does not depend on what else is in the batch.
#include "tw_common.h"
#include "tw_sampling.h"

#include <mutex>

__host__ __device__ static inline uint64_t tw_splitmix64(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

// Uniform in [0, 1) with 23 random bits, so that u * total < total in float32.
__host__ __device__ static inline float tw_uniform(uint64_t seed, uint64_t counter) {
  const uint64_t bits = tw_splitmix64(tw_splitmix64(seed) + counter);
  return (float)(bits >> 41) * (1.0f / 8388608.0f);
}

extern "C" float tw_sampling_uniform(uint64_t seed, uint64_t counter) { return tw_uniform(seed, counter); }

// Two kernels, so that a handful of rows still use the whole chip: the vocabulary is cut into
// TW_SAMPLE_CHUNKS chunks; `sample_scan` reduces every (row, chunk) to its largest logit, the
// lowest index where it stands and (for sampling) sum exp((x - chunk max) / T); `sample_pick`
// merges a row's chunks in index order, draws the chunk and rescans only that chunk for the id.
#define TW_SAMPLE_CHUNKS 64
#define TW_SAMPLE_THREADS 256

struct SamplePartial {
  float max;
  int arg;
  float sum;     // sum over the chunk of exp((x - max) / T); 0 for greedy rows
  float pad;
};

__device__ __forceinline__ int tw_sample_chunk_width(int vocab) {
  return (vocab + TW_SAMPLE_CHUNKS - 1) / TW_SAMPLE_CHUNKS;
}

__global__ __launch_bounds__(TW_SAMPLE_THREADS) void sample_scan_kernel(
    const float* __restrict__ logits, long ld, int vocab, const float* __restrict__ temperature,
    SamplePartial* __restrict__ partial) {
  __shared__ float s_val[TW_SAMPLE_THREADS];
  __shared__ int s_idx[TW_SAMPLE_THREADS];
  const int chunk = blockIdx.x, row = blockIdx.y, tid = threadIdx.x;
  const float* x = logits + (size_t)row * ld;
  const int width = tw_sample_chunk_width(vocab);
  const int begin = min(vocab, chunk * width), end = min(vocab, begin + width);
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for (int i = begin + tid; i < end; i += TW_SAMPLE_THREADS) {
    const float v = x[i];
    if (v > best) { best = v; best_i = i; }       // strided: earlier i seen first
  }
  s_val[tid] = best;
  s_idx[tid] = best_i;
  __syncthreads();
  for (int stride = TW_SAMPLE_THREADS / 2; stride > 0; stride >>= 1) {
    if (tid < stride) {
      const float ov = s_val[tid + stride];
      const int oi = s_idx[tid + stride];
      if (ov > s_val[tid] || (ov == s_val[tid] && oi < s_idx[tid])) { s_val[tid] = ov; s_idx[tid] = oi; }
    }
    __syncthreads();
  }
  const float mx = s_val[0];
  const int arg = s_idx[0];
  const float temp = temperature ? temperature[row] : 0.f;
  float total = 0.f;
  if (temp > 0.f && end > begin) {
    __syncthreads();
    const float inv_t = 1.0f / temp;
    float mine = 0.f;
    for (int i = begin + tid; i < end; i += TW_SAMPLE_THREADS) mine += expf((x[i] - mx) * inv_t);
    s_val[tid] = mine;
    __syncthreads();
    for (int stride = TW_SAMPLE_THREADS / 2; stride > 0; stride >>= 1) {    // a fixed tree: same sum every time
      if (tid < stride) s_val[tid] += s_val[tid + stride];
      __syncthreads();
    }
    total = s_val[0];
  }
  if (tid == 0) {
    SamplePartial p;
    p.max = mx; p.arg = arg; p.sum = total; p.pad = 0.f;
    partial[(size_t)row * TW_SAMPLE_CHUNKS + chunk] = p;
  }
}

__global__ __launch_bounds__(TW_SAMPLE_THREADS) void sample_pick_kernel(
    const float* __restrict__ logits, long ld, int vocab, const float* __restrict__ temperature,
    const uint64_t* __restrict__ seeds, const int* __restrict__ counters,
    const SamplePartial* __restrict__ partial, int* __restrict__ out) {
  __shared__ float s_val[TW_SAMPLE_THREADS];
  __shared__ int s_pick[2];
  __shared__ float s_before;
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)row * ld;
  const SamplePartial* part = partial + (size_t)row * TW_SAMPLE_CHUNKS;

  // ---- largest logit, lowest index on ties (chunks are in index order) -----------
  float mx = -INFINITY;
  int arg = 0x7fffffff;
  for (int c = 0; c < TW_SAMPLE_CHUNKS; ++c) {
    const float v = part[c].max;
    if (v > mx) { mx = v; arg = part[c].arg; }
  }
  if (arg == 0x7fffffff) arg = 0;
  const float temp = temperature ? temperature[row] : 0.f;
  if (!(temp > 0.f)) {
    if (tid == 0) out[row] = arg;
    return;
  }
  // ---- which chunk: inverse CDF over the chunks' weights, summed in index order ----
  const float inv_t = 1.0f / temp;
  if (tid == 0) {
    float total = 0.f;
    for (int c = 0; c < TW_SAMPLE_CHUNKS; ++c) total += part[c].sum * expf((part[c].max - mx) * inv_t);
    int chunk = -1;
    float before = 0.f;
    if (total > 0.f && !isinf(total)) {
      const float target = tw_uniform(seeds[row], (uint64_t)(uint32_t)counters[row]) * total;
      float run = 0.f;
      int last = -1;
      for (int c = 0; c < TW_SAMPLE_CHUNKS; ++c) {
        const float w = part[c].sum * expf((part[c].max - mx) * inv_t);
        if (w > 0.f) last = c;
        if (run + w > target) { chunk = c; before = run; break; }
        run += w;
      }
      if (chunk < 0) { chunk = last; before = target; }        // rounding: the last chunk that has weight
      s_before = target - before;                               // what is left to cross inside the chunk
    }
    s_pick[0] = chunk;
  }
  __syncthreads();
  const int chunk = s_pick[0];
  if (chunk < 0) {                                   // not a distribution (NaN or overflow): fall back to greedy
    if (tid == 0) out[row] = arg;
    return;
  }
  // ---- which id inside the chunk: contiguous pieces per thread, scanned in order ----
  const float target = s_before;
  const int width = tw_sample_chunk_width(vocab);
  const int cb = min(vocab, chunk * width), ce = min(vocab, cb + width);
  const int piece = (ce - cb + TW_SAMPLE_THREADS - 1) / TW_SAMPLE_THREADS;
  const int begin = min(ce, cb + tid * piece), end = min(ce, begin + piece);
  float mine = 0.f;
  for (int i = begin; i < end; ++i) mine += expf((x[i] - mx) * inv_t);
  s_val[tid] = mine;
  __syncthreads();
  if (tid == 0) {
    float run = 0.f;
    int owner = -1, last = 0;
    for (int i = 0; i < TW_SAMPLE_THREADS; ++i) {
      if (s_val[i] > 0.f) last = i;
      if (owner < 0 && run + s_val[i] > target) { owner = i; s_before = run; }
      run += s_val[i];
    }
    if (owner < 0) { owner = last; s_before = target; }        // rounding: the last piece that has weight
    s_pick[1] = owner;
  }
  __syncthreads();
  if (tid == s_pick[1]) {
    float run = s_before;
    int pick = -1, last = begin;
    for (int i = begin; i < end; ++i) {
      const float e = expf((x[i] - mx) * inv_t);
      if (e > 0.f) last = i;
      run += e;
      if (run > target) { pick = i; break; }
    }
    out[row] = pick >= 0 ? pick : last;
  }
}

static int sample_launch(const float* logits, long ld, int rows, int vocab, const float* temperature,
                         const uint64_t* seeds, const int* counters, int* out, SamplePartial* partial,
                         hipStream_t stream) {
  sample_scan_kernel<<<dim3(TW_SAMPLE_CHUNKS, rows), TW_SAMPLE_THREADS, 0, stream>>>(logits, ld, vocab, temperature, partial);
  int err = TW_LAUNCH_RESULT();
  if (err) return err;
  sample_pick_kernel<<<rows, TW_SAMPLE_THREADS, 0, stream>>>(logits, ld, vocab, temperature, seeds, counters, partial, out);
  return TW_LAUNCH_RESULT();
}

extern "C" long tw_sample_workspace_bytes(int rows) { return (long)rows * TW_SAMPLE_CHUNKS * sizeof(SamplePartial); }

// logits [rows][ld] float32; temperature (may be null: all greedy), seeds, counters per row;
// workspace: tw_sample_workspace_bytes(rows) bytes of scratch.
extern "C" int tw_sample_rows(const float* logits, long ld, int rows, int vocab, const float* temperature,
                              const uint64_t* seeds, const int* counters, int* out, void* workspace,
                              long workspace_bytes, hipStream_t stream) {
  TW_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab && rows <= 65535);
  TW_REQUIRE(temperature == nullptr || (seeds != nullptr && counters != nullptr));
  if (rows == 0) return 0;
  TW_REQUIRE(workspace != nullptr && workspace_bytes >= tw_sample_workspace_bytes(rows) && (uintptr_t)workspace % 16 == 0);
  return sample_launch(logits, ld, rows, vocab, temperature, seeds, counters, out, (SamplePartial*)workspace, stream);
}

// ---- the same without a workspace from the caller: partial results in the library's own device image ----
// `scratch` is a name of HOST code here: the device address behind it differs per GPU and is looked up
// once per device (below); kernels only ever get that looked-up pointer.
static __device__ __align__(256) unsigned char scratch[TW_SAMPLE_STATIC_MAX_ROWS * TW_SAMPLE_CHUNKS * sizeof(SamplePartial)];

#define TW_SAMPLE_MAX_DEVICES 64
static void* g_scratch_of_device[TW_SAMPLE_MAX_DEVICES];
static std::mutex g_scratch_mutex;

// The address of `scratch` on the CURRENT device, looked up on the first call there.
static int scratch_on_current_device(void** out) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return (int)e;
  if (device < 0 || device >= TW_SAMPLE_MAX_DEVICES) return TW_ERR_BAD_ARGUMENT;
  std::lock_guard<std::mutex> guard(g_scratch_mutex);
  if (g_scratch_of_device[device] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (ptr == nullptr) return (int)hipErrorInvalidSymbol;
    g_scratch_of_device[device] = ptr;
  }
  *out = g_scratch_of_device[device];
  return 0;
}

extern "C" int tw_sample_rows_static(const float* logits, long ld, int rows, int vocab, const float* temperature,
                                     const uint64_t* seeds, const int* counters, int* out, hipStream_t stream) {
  TW_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab);
  TW_REQUIRE(temperature == nullptr || (seeds != nullptr && counters != nullptr));
  if (rows > TW_SAMPLE_STATIC_MAX_ROWS) return TW_ERR_TOO_LARGE;
  if (rows == 0) return 0;
  void* partial = nullptr;
  const int err = scratch_on_current_device(&partial);
  if (err) return err;
  return sample_launch(logits, ld, rows, vocab, temperature, seeds, counters, out, (SamplePartial*)partial, stream);
}
