// Next-token choice per logits row: greedy (temperature 0: the lowest index among
// the largest logits) or temperature sampling by inverse CDF over
// softmax(logits / T), all in float32. The uniform number of a row comes from a
// counter-based generator keyed by (the request's seed, the index of the token
// being drawn), so a request's stream does not depend on what else is in the batch.
#include "tw_common.h"

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

#define TW_SAMPLE_THREADS 1024

__global__ __launch_bounds__(TW_SAMPLE_THREADS) void sample_rows_kernel(
    const float* __restrict__ logits, long ld, int vocab, const float* __restrict__ temperature,
    const uint64_t* __restrict__ seeds, const int* __restrict__ counters, int* __restrict__ out) {
  __shared__ float s_val[TW_SAMPLE_THREADS];
  __shared__ int s_idx[TW_SAMPLE_THREADS];
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)row * ld;

  // ---- largest logit, lowest index on ties -------------------------------------
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for (int i = tid; i < vocab; i += TW_SAMPLE_THREADS) {
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
  const int arg = s_idx[0] == 0x7fffffff ? 0 : s_idx[0];
  const float temp = temperature ? temperature[row] : 0.f;
  if (!(temp > 0.f)) {
    if (tid == 0) out[row] = arg;
    return;
  }
  __syncthreads();

  // ---- inverse CDF over exp((x - max) / T), contiguous chunk per thread --------
  const float inv_t = 1.0f / temp;
  const int chunk = (vocab + TW_SAMPLE_THREADS - 1) / TW_SAMPLE_THREADS;
  const int begin = min(vocab, tid * chunk), end = min(vocab, begin + chunk);
  float mine = 0.f;
  for (int i = begin; i < end; ++i) mine += expf((x[i] - mx) * inv_t);
  s_val[tid] = mine;
  __syncthreads();
  if (tid == 0) {
    float run = 0.f;
    for (int i = 0; i < TW_SAMPLE_THREADS; ++i) { run += s_val[i]; s_val[i] = run; }   // inclusive scan, fixed order
  }
  __syncthreads();
  const float total = s_val[TW_SAMPLE_THREADS - 1];
  if (!(total > 0.f) || isinf(total)) {            // not a distribution (NaN or overflow): fall back to greedy
    if (tid == 0) out[row] = arg;
    return;
  }
  const float target = tw_uniform(seeds[row], (uint64_t)(uint32_t)counters[row]) * total;
  const float before = tid == 0 ? 0.f : s_val[tid - 1];
  const float upto = s_val[tid];
  if (target >= before && target < upto && end > begin) {
    float run = before;
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

// logits [rows][ld] float32; temperature (may be null: all greedy), seeds, counters per row.
extern "C" int tw_sample_rows(const float* logits, long ld, int rows, int vocab, const float* temperature,
                              const uint64_t* seeds, const int* counters, int* out, hipStream_t stream) {
  TW_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab);
  TW_REQUIRE(temperature == nullptr || (seeds != nullptr && counters != nullptr));
  if (rows == 0) return 0;
  sample_rows_kernel<<<rows, TW_SAMPLE_THREADS, 0, stream>>>(logits, ld, vocab, temperature, seeds, counters, out);
  return TW_LAUNCH_RESULT();
}
