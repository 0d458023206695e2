// Row kernels: embedding gather, RMS norm, rotary tables, rotation + cache
// write, SiLU-multiply. Statistics, angles and products are float32; storage
// is float32 or bfloat16. The residual stream is float32 in both precisions.
#include "tw_common.h"

// ---- embedding: x[n, :] = float(E[ids[n], :]) ------------------------------------
// A negative id -1 - k stands for feed[k]: a token that an earlier kernel on this stream wrote
// (the sampler's output of the step before), which the host has not read yet.
template <typename T>
__global__ void embed_gather_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                    float* __restrict__ out, int hidden, int vocab,
                                    const int* __restrict__ feed, int feed_count) {
  const int n = blockIdx.x;
  int id = ids[n];
  if (id < 0 && feed != nullptr && -1 - id < feed_count) id = feed[-1 - id];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);   // ids are validated on the host; never read outside
  const T* row = table + (size_t)id * hidden;
  float* dst = out + (size_t)n * hidden;
  for (int h = threadIdx.x; h < hidden; h += blockDim.x) dst[h] = tw_to_float(row[h]);
}

extern "C" int tw_embed_gather(int dtype, const int* ids, const void* table, float* out, int n,
                               int hidden, int vocab, const int* feed, int feed_count, hipStream_t stream) {
  TW_REQUIRE(n >= 0 && hidden > 0 && vocab > 0 && feed_count >= 0);
  if (n == 0) return 0;
  if (dtype == TW_DTYPE_F32)
    embed_gather_kernel<float><<<n, 256, 0, stream>>>(ids, (const float*)table, out, hidden, vocab, feed, feed_count);
  else if (dtype == TW_DTYPE_BF16)
    embed_gather_kernel<bf16_t><<<n, 256, 0, stream>>>(ids, (const bf16_t*)table, out, hidden, vocab, feed, feed_count);
  else
    return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}

// ---- RMS norm -------------------------------------------------------------------------
// y = x * rsqrt(mean(x^2) + eps) * w, statistics and products in float32, one
// rounding to the output type. `rows` (optional) picks the input row of each
// output row. If `add` is given the input row is (sum_s add[s]) + x (split-K
// partial sums of the layer before, added up in the order the separate
// reduction kernel uses); without `rows` that sum is also written back to x.
template <typename T>
__global__ void rmsnorm_kernel(float* __restrict__ x, const float* __restrict__ w, T* __restrict__ out,
                               const int* __restrict__ rows, int hidden, float eps,
                               const float* __restrict__ add, int add_splits, size_t add_stride,
                               float* __restrict__ row_scratch) {
  __shared__ float lds[16];
  const int o = blockIdx.x;
  const int r = rows ? rows[o] : o;
  float* src = x + (size_t)r * hidden;
  float ss = 0.f;
  if (add) {
    // with gathered rows the sums go to a scratch row (two outputs may name one input row)
    float* dst = rows ? row_scratch + (size_t)o * hidden : src;
    for (int h = threadIdx.x; h < hidden; h += blockDim.x) {
      float v = 0.f;
      for (int s = 0; s < add_splits; ++s) v += add[s * add_stride + (size_t)r * hidden + h];
      v += src[h];
      dst[h] = v;
      ss += v * v;
    }
    src = dst;
  } else {
    for (int h = threadIdx.x; h < hidden; h += blockDim.x) {
      const float v = src[h];
      ss += v * v;
    }
  }
  ss = tw_block_sum(ss, lds);
  const float scale = 1.0f / sqrtf(ss / (float)hidden + eps);
  T* dst = out + (size_t)o * hidden;
  for (int h = threadIdx.x; h < hidden; h += blockDim.x)
    dst[h] = tw_from_float<T>(src[h] * scale * w[h]);
}

// The same for hidden % 4 == 0 with at most 4 * G * blockDim.x elements per row: every
// thread owns G groups of 4 consecutive elements (blockDim.x groups apart), kept in registers
// between the two passes; the partial sums are read with independent 16-byte loads. (The sum
// of squares is associated differently from the kernel above: results of the two
// kernels agree to rounding, not to the bit.)
template <typename T, int G>
__global__ void rmsnorm_vec4_kernel(float* __restrict__ x, const float* __restrict__ w, T* __restrict__ out,
                                    const int* __restrict__ rows, int hidden, float eps,
                                    const float* __restrict__ add, int add_splits, size_t add_stride) {
  __shared__ float lds[16];
  const int o = blockIdx.x;
  const int r = rows ? rows[o] : o;
  float* src = x + (size_t)r * hidden;
  f32x4 v[G], wv[G], xv[G];
  int h[G];
  bool mine[G];
  // Every load of the row is issued before the first one is waited for (the kernel's time is a
  // chain of memory latencies): the row itself, the weight, and the partial sums 8 at a time.
  // The partial sums are still added one after the other in index order, then the row.
#pragma unroll
  for (int gi = 0; gi < G; ++gi) {
    h[gi] = (gi * (int)blockDim.x + (int)threadIdx.x) * 4;
    mine[gi] = h[gi] < hidden;
    v[gi] = f32x4{0.f, 0.f, 0.f, 0.f};
    wv[gi] = f32x4{0.f, 0.f, 0.f, 0.f};
    xv[gi] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (mine[gi]) {
      xv[gi] = *reinterpret_cast<const f32x4*>(src + h[gi]);
      if (add) wv[gi] = *reinterpret_cast<const f32x4*>(w + h[gi]);   // (few rows; with many, the weight is read below)
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int gi = 0; gi < G; ++gi) {
    if (mine[gi]) {
      if (add) {
        const float* p = add + (size_t)r * hidden + h[gi];
        for (int s0 = 0; s0 < add_splits; s0 += 8) {
          f32x4 a[8];
#pragma unroll
          for (int i = 0; i < 8; ++i)
            a[i] = s0 + i < add_splits ? *reinterpret_cast<const f32x4*>(p + (size_t)(s0 + i) * add_stride)
                                       : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int i = 0; i < 8; ++i)
            if (s0 + i < add_splits) v[gi] = v[gi] + a[i];
        }
        v[gi] = v[gi] + xv[gi];
        if (!rows) *reinterpret_cast<f32x4*>(src + h[gi]) = v[gi];
      } else {
        v[gi] = xv[gi];
      }
      ss += ((v[gi][0] * v[gi][0] + v[gi][1] * v[gi][1]) + v[gi][2] * v[gi][2]) + v[gi][3] * v[gi][3];
    }
  }
  ss = tw_block_sum(ss, lds);
  const float scale = 1.0f / sqrtf(ss / (float)hidden + eps);
#pragma unroll
  for (int gi = 0; gi < G; ++gi) {
    if (!mine[gi]) continue;
    if (!add) wv[gi] = *reinterpret_cast<const f32x4*>(w + h[gi]);
    T* dst = out + (size_t)o * hidden + h[gi];
    T packed[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) packed[e] = tw_from_float<T>(v[gi][e] * scale * wv[gi][e]);
    if (sizeof(T) == 2 && ((uintptr_t)out % 8 == 0))
      *reinterpret_cast<uint64_t*>(dst) = *reinterpret_cast<const uint64_t*>(packed);      // hidden % 4 == 0: aligned
    else if (sizeof(T) == 4 && ((uintptr_t)out % 16 == 0))
      *reinterpret_cast<f32x4*>(dst) = *reinterpret_cast<const f32x4*>(packed);
    else {
#pragma unroll
      for (int e = 0; e < 4; ++e) dst[e] = packed[e];
    }
  }
}

// Many rows: one WAVE per row (4 rows per workgroup), a row of up to 256 * NG elements in registers as
// up to NG groups of 4, every load of a pass issued at once, and no barrier: the sum of squares is a wave
// reduction. (With one workgroup of 896 threads per row, 2,048 rows of 3,584 took 15 us.) With ADD the
// row is (sum_s add[s]) + x, added in that order as everywhere, and written back to x.
template <typename T, int NG, bool ADD>
__global__ __launch_bounds__(256) void rmsnorm_wave_kernel(float* __restrict__ x, const float* __restrict__ w,
                                                           T* __restrict__ out, int n_rows, int hidden, float eps,
                                                           const float* __restrict__ add, int add_splits,
                                                           size_t add_stride) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= n_rows) return;
  float* src = x + (size_t)row * hidden;
  f32x4 v[NG];
  float ss = 0.f;
  if (ADD) {
    // CH groups at a time (a whole row of up to 4,096 elements, half of a longer one): the row's own
    // values and one split's sums are in flight together
    constexpr int CH = NG <= 16 ? NG : 16;
    const float* p = add + (size_t)row * hidden;
#pragma unroll
    for (int c = 0; c < NG; c += CH) {
      f32x4 xv[CH], acc[CH];
#pragma unroll
      for (int j = 0; j < CH; ++j) {
        const int h = ((c + j) * 64 + lane) * 4;
        xv[j] = h < hidden ? *reinterpret_cast<const f32x4*>(src + h) : f32x4{0.f, 0.f, 0.f, 0.f};
        acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
      for (int s = 0; s < add_splits; ++s) {
        f32x4 a[CH];
#pragma unroll
        for (int j = 0; j < CH; ++j) {
          const int h = ((c + j) * 64 + lane) * 4;
          a[j] = h < hidden ? *reinterpret_cast<const f32x4*>(p + s * add_stride + h) : f32x4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int j = 0; j < CH; ++j) acc[j] = acc[j] + a[j];
      }
#pragma unroll
      for (int j = 0; j < CH; ++j) {
        const int h = ((c + j) * 64 + lane) * 4;
        v[c + j] = acc[j] + xv[j];
        if (h < hidden) *reinterpret_cast<f32x4*>(src + h) = v[c + j];
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < NG; ++i) {
      const int h = (i * 64 + lane) * 4;
      v[i] = h < hidden ? *reinterpret_cast<const f32x4*>(src + h) : f32x4{0.f, 0.f, 0.f, 0.f};
    }
  }
#pragma unroll
  for (int i = 0; i < NG; ++i) ss += ((v[i][0] * v[i][0] + v[i][1] * v[i][1]) + v[i][2] * v[i][2]) + v[i][3] * v[i][3];
  ss = tw_wave_sum(ss);
  const float scale = 1.0f / sqrtf(ss / (float)hidden + eps);
  T* dst = out + (size_t)row * hidden;
#pragma unroll
  for (int i = 0; i < NG; ++i) {
    const int h = (i * 64 + lane) * 4;
    if (h >= hidden) continue;
    const f32x4 wv = *reinterpret_cast<const f32x4*>(w + h);
    T packed[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) packed[e] = tw_from_float<T>(v[i][e] * scale * wv[e]);
    if (sizeof(T) == 2)
      *reinterpret_cast<uint64_t*>(dst + h) = *reinterpret_cast<const uint64_t*>(packed);
    else
      *reinterpret_cast<f32x4*>(dst + h) = *reinterpret_cast<const f32x4*>(packed);
  }
}

template <typename T>
static void launch_rmsnorm_vec4(int groups_per_thread, int n_out, int threads, hipStream_t stream, float* x,
                                const float* w, T* out, const int* rows, int hidden, float eps, const float* add,
                                int add_splits, size_t add_stride) {
  if (groups_per_thread == 1)
    rmsnorm_vec4_kernel<T, 1><<<n_out, threads, 0, stream>>>(x, w, out, rows, hidden, eps, add, add_splits, add_stride);
  else if (groups_per_thread == 2)
    rmsnorm_vec4_kernel<T, 2><<<n_out, threads, 0, stream>>>(x, w, out, rows, hidden, eps, add, add_splits, add_stride);
  else
    rmsnorm_vec4_kernel<T, 4><<<n_out, threads, 0, stream>>>(x, w, out, rows, hidden, eps, add, add_splits, add_stride);
}

template <typename T>
static void launch_rmsnorm_wave(int n_out, hipStream_t stream, float* x, const float* w, T* out, int hidden,
                                float eps, const float* add, int add_splits, size_t add_stride) {
  const int grid = (n_out + 3) / 4;
  if (hidden <= 4096) {
    if (add) rmsnorm_wave_kernel<T, 16, true><<<grid, 256, 0, stream>>>(x, w, out, n_out, hidden, eps, add, add_splits, add_stride);
    else rmsnorm_wave_kernel<T, 16, false><<<grid, 256, 0, stream>>>(x, w, out, n_out, hidden, eps, nullptr, 0, 0);
  } else {
    if (add) rmsnorm_wave_kernel<T, 32, true><<<grid, 256, 0, stream>>>(x, w, out, n_out, hidden, eps, add, add_splits, add_stride);
    else rmsnorm_wave_kernel<T, 32, false><<<grid, 256, 0, stream>>>(x, w, out, n_out, hidden, eps, nullptr, 0, 0);
  }
}

extern "C" int tw_rmsnorm(int out_dtype, float* x, const float* w, void* out, const int* rows,
                          int n_out, int hidden, float eps, const float* add, int add_splits,
                          long add_stride, float* row_scratch, hipStream_t stream) {
  TW_REQUIRE(n_out >= 0 && hidden > 0 && eps > 0.f);
  TW_REQUIRE(add == nullptr || (add_splits > 0 && (rows == nullptr || row_scratch != nullptr)));
  if (n_out == 0) return 0;
  if (out_dtype != TW_DTYPE_F32 && out_dtype != TW_DTYPE_BF16) return TW_ERR_BAD_ARGUMENT;
  if (rows == nullptr && n_out >= 256 && hidden % 4 == 0 && hidden <= 8192 &&
      (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0 && (uintptr_t)out % 16 == 0 &&
      (add == nullptr || ((uintptr_t)add % 16 == 0 && add_stride % 4 == 0))) {
    if (out_dtype == TW_DTYPE_F32)
      launch_rmsnorm_wave<float>(n_out, stream, x, w, (float*)out, hidden, eps, add, add_splits, (size_t)add_stride);
    else
      launch_rmsnorm_wave<bf16_t>(n_out, stream, x, w, (bf16_t*)out, hidden, eps, add, add_splits, (size_t)add_stride);
    return TW_LAUNCH_RESULT();
  }
  // rows of up to 16384 elements: one, two or four groups of 4 elements per thread, everything in registers
  if (hidden % 4 == 0 && hidden <= 16384 && (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0 &&
      (add == nullptr || ((uintptr_t)add % 16 == 0 && add_stride % 4 == 0))) {
    const int per_thread = hidden <= 4096 ? 1 : (hidden <= 8192 ? 2 : 4);
    const int threads = (hidden / 4 + per_thread * 64 - 1) / (per_thread * 64) * 64;
    if (out_dtype == TW_DTYPE_F32)
      launch_rmsnorm_vec4<float>(per_thread, n_out, threads, stream, x, w, (float*)out, rows, hidden, eps, add,
                                 add_splits, (size_t)add_stride);
    else
      launch_rmsnorm_vec4<bf16_t>(per_thread, n_out, threads, stream, x, w, (bf16_t*)out, rows, hidden, eps, add,
                                  add_splits, (size_t)add_stride);
    return TW_LAUNCH_RESULT();
  }
  const int threads = hidden >= 2048 ? 512 : 256;
  if (out_dtype == TW_DTYPE_F32)
    rmsnorm_kernel<float><<<n_out, threads, 0, stream>>>(x, w, (float*)out, rows, hidden, eps, add,
                                                         add_splits, (size_t)add_stride, row_scratch);
  else
    rmsnorm_kernel<bf16_t><<<n_out, threads, 0, stream>>>(x, w, (bf16_t*)out, rows, hidden, eps, add,
                                                          add_splits, (size_t)add_stride, row_scratch);
  return TW_LAUNCH_RESULT();
}

// ---- rotary tables: cos/sin[n, j] of angle = float(position[n]) * inv_freq[j] -----
__global__ void rope_table_kernel(const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                  float* __restrict__ cos_out, float* __restrict__ sin_out, int n, int half) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n * half) return;
  const int t = i / half, j = i % half;
  const float angle = (float)positions[t] * inv_freq[j];
  cos_out[i] = cosf(angle);
  sin_out[i] = sinf(angle);
}

extern "C" int tw_rope_table(const int* positions, const float* inv_freq, float* cos_out, float* sin_out,
                             int n, int half, hipStream_t stream) {
  TW_REQUIRE(n >= 0 && half > 0);
  if (n == 0) return 0;
  rope_table_kernel<<<tw_div_up((long)n * half, 256), 256, 0, stream>>>(positions, inv_freq, cos_out,
                                                                       sin_out, n, half);
  return TW_LAUNCH_RESULT();
}

// ---- rotation of q and k, and the cache write ----------------------------------------------
// qkv[n] = [q heads | k heads | v heads], head-major, `ld` elements per row.
// Pair j of a head is (x[j], x[j + rot/2]) for j < rot/2 (rotate-half), or, with `adjacent`,
// (x[2j], x[2j + 1]); elements from `rot` on are not rotated. q is rotated in place. Rotated k goes to
//   keys  [page][kv_head][offset][d]      and raw v to
//   values[page][kv_head][d][offset]      (transposed inside the page),
// slot = page * page_size + offset; a negative slot writes nothing.
// (With `partial`, the split-K sums of the q/k/v projection, qkv_finish_kernel below does the
// same from round_T(sum_s partial[s][n][col] + bias[col]), one workgroup per (token, head).)
// One rotated pair, with the products and sums spelled out so that both kernels below round alike
// (left to the compiler, a*b - c*d is contracted to one fused multiply-add or the other).
__device__ __forceinline__ void tw_rotate_pair(float lo, float hi, float c, float s, float& out_lo, float& out_hi) {
  out_lo = __fmaf_rn(lo, c, -__fmul_rn(hi, s));
  out_hi = __fmaf_rn(hi, c, __fmul_rn(lo, s));
}

template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, long ld, const float* __restrict__ cos_t,
                                     const float* __restrict__ sin_t, const int* __restrict__ slots,
                                     T* __restrict__ keys, T* __restrict__ values, int q_heads,
                                     int kv_heads, int head_dim, int rot, int page_size, int write_cache,
                                     int adjacent) {
  const int n = blockIdx.x;
  const int half = rot / 2;
  T* row = qkv + (size_t)n * ld;
  const float* c = cos_t + (size_t)n * half;
  const float* s = sin_t + (size_t)n * half;
  const int slot = write_cache ? slots[n] : -1;
  const int page = slot >= 0 ? slot / page_size : 0;
  const int off = slot >= 0 ? slot % page_size : 0;
  const int rot_heads = q_heads + kv_heads;
  // rotated part: one thread per pair
  for (int i = threadIdx.x; i < rot_heads * half; i += blockDim.x) {
    const int head = i / half, j = i % half;
    T* x = row + (size_t)head * head_dim;
    const int i_lo = adjacent ? 2 * j : j, i_hi = adjacent ? 2 * j + 1 : j + half;
    const float lo = tw_to_float(x[i_lo]), hi = tw_to_float(x[i_hi]);
    float r_lo, r_hi;
    tw_rotate_pair(lo, hi, c[j], s[j], r_lo, r_hi);
    const T out_lo = tw_from_float<T>(r_lo), out_hi = tw_from_float<T>(r_hi);
    if (head < q_heads) {
      x[i_lo] = out_lo;
      x[i_hi] = out_hi;
    } else if (slot >= 0) {
      const int kh = head - q_heads;
      T* dst = keys + (((size_t)page * kv_heads + kh) * page_size + off) * head_dim;
      dst[i_lo] = out_lo;
      dst[i_hi] = out_hi;
    }
  }
  if (slot < 0) return;
  // unrotated tail of the keys
  const int tail = head_dim - rot;
  for (int i = threadIdx.x; i < kv_heads * tail; i += blockDim.x) {
    const int kh = i / tail, d = rot + i % tail;
    keys[(((size_t)page * kv_heads + kh) * page_size + off) * head_dim + d] =
        row[(size_t)(q_heads + kh) * head_dim + d];
  }
  // values, transposed inside the page
  const T* v = row + (size_t)(q_heads + kv_heads) * head_dim;
  for (int i = threadIdx.x; i < kv_heads * head_dim; i += blockDim.x) {
    const int kh = i / head_dim, d = i % head_dim;
    values[(((size_t)page * kv_heads + kh) * head_dim + d) * page_size + off] = v[i];
  }
}

// The same work from split-K partial sums, one workgroup per (token, head): the
// head's values are round_T(sum_s partial[s][n][col] + bias[col]); q heads are
// rotated into qkv, k heads are rotated into the pages, v heads go to the pages.
// The common case of rope_kv_write_kernel (the whole head rotated as pairs (j, j + half), every row and
// pointer 16-byte aligned): a thread moves 16 bytes of each half of a head at a time, and finds its head
// with one division instead of one per element. Every element goes through the same arithmetic, so the
// two kernels give the same bits. (2,048 tokens of 36 heads of 128, cold: the rotation alone 12.5 -> 7.7 us;
// with the cache written 18.4 -> 14.9 us, of which the grouped stores of the values, below, are 1.3.)
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_write_vec_kernel(T* __restrict__ qkv, long ld,
                                                                const float* __restrict__ cos_t,
                                                                const float* __restrict__ sin_t,
                                                                const int* __restrict__ slots, T* __restrict__ keys,
                                                                T* __restrict__ values, int q_heads, int kv_heads,
                                                                int head_dim, int page_size, int write_cache) {
  typedef typename Elem<T>::Frag Frag;
  constexpr int V = Elem<T>::kPerFrag;
  const int n = blockIdx.x;
  const int half = head_dim / 2, cpb = half / V;             // 16-byte chunks per half head
  T* row = qkv + (size_t)n * ld;
  const float* c = cos_t + (size_t)n * half;
  const float* s = sin_t + (size_t)n * half;
  const int slot = write_cache ? slots[n] : -1;
  const int page = slot >= 0 ? slot / page_size : 0;
  const int off = slot >= 0 ? slot % page_size : 0;
  const int rot_heads = q_heads + kv_heads;
  for (int item = threadIdx.x; item < rot_heads * cpb; item += blockDim.x) {
    const int head = item / cpb, j0 = (item - head * cpb) * V;
    T* x = row + (size_t)head * head_dim;
    T* dst = x;
    if (head >= q_heads) {
      if (slot < 0) continue;
      dst = keys + (((size_t)page * kv_heads + (head - q_heads)) * page_size + off) * head_dim;
    }
    const Frag lo = tw_load_frag(x + j0), hi = tw_load_frag(x + half + j0);
    float cj[V], sj[V];
#pragma unroll
    for (int q = 0; q < V / 4; ++q) {
      const f32x4 cq = *reinterpret_cast<const f32x4*>(c + j0 + 4 * q);
      const f32x4 sq = *reinterpret_cast<const f32x4*>(s + j0 + 4 * q);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        cj[4 * q + e] = cq[e];
        sj[4 * q + e] = sq[e];
      }
    }
    Frag out_lo, out_hi;
#pragma unroll
    for (int e = 0; e < V; ++e) {
      float r_lo, r_hi;
      tw_rotate_pair(tw_to_float(lo[e]), tw_to_float(hi[e]), cj[e], sj[e], r_lo, r_hi);
      out_lo[e] = tw_from_float<T>(r_lo);
      out_hi[e] = tw_from_float<T>(r_hi);
    }
    *reinterpret_cast<Frag*>(dst + j0) = out_lo;
    *reinterpret_cast<Frag*>(dst + half + j0) = out_hi;
  }
  if (slot < 0) return;
  // Values, transposed inside the page: element (head, d) of this token goes to [d][off], so a token alone
  // writes one element at a time. Where V tokens in a row of the batch hold V consecutive slots that start
  // at a multiple of V (a prompt portion: 16 bytes of one [d] row of the page), the first of them writes
  // for all and the others write nothing: each thread reads 16 bytes of each token's row and stores V
  // vectors of V tokens. Every token of such a group sees the same slots and decides alike.
  const int vpb = head_dim / V;
  const int lead = n - off % V;
  bool grouped = page_size % V == 0 && lead >= 0 && lead + V <= (int)gridDim.x;
  if (grouped) {
    const int first = slots[lead];
    grouped = first >= 0 && first == slot - off % V;
#pragma unroll
    for (int i = 1; i < V; ++i) grouped = grouped && slots[lead + i] == first + i;
  }
  if (grouped) {
    if (n != lead) return;
    const T* v0 = row + (size_t)rot_heads * head_dim;                  // this (the first) token's values
    for (int item = threadIdx.x; item < kv_heads * vpb; item += blockDim.x) {
      const int kh = item / vpb, d0 = (item - kh * vpb) * V;
      Frag val[V];
#pragma unroll
      for (int i = 0; i < V; ++i) val[i] = tw_load_frag(v0 + (size_t)i * ld + (size_t)kh * head_dim + d0);
      T* dst = values + (((size_t)page * kv_heads + kh) * head_dim + d0) * page_size + off;
#pragma unroll
      for (int e = 0; e < V; ++e) {
        Frag column;
#pragma unroll
        for (int i = 0; i < V; ++i) column[i] = val[i][e];
        *reinterpret_cast<Frag*>(dst + (size_t)e * page_size) = column;
      }
    }
    return;
  }
  const T* v = row + (size_t)rot_heads * head_dim;
  for (int item = threadIdx.x; item < kv_heads * vpb; item += blockDim.x) {
    const int kh = item / vpb, d0 = (item - kh * vpb) * V;
    const Frag val = tw_load_frag(v + (size_t)kh * head_dim + d0);
    T* dst = values + (((size_t)page * kv_heads + kh) * head_dim + d0) * page_size + off;
#pragma unroll
    for (int e = 0; e < V; ++e) dst[(size_t)e * page_size] = val[e];
  }
}

template <typename T>
__global__ void qkv_finish_kernel(T* __restrict__ qkv, long ld, const float* __restrict__ cos_t,
                                  const float* __restrict__ sin_t, const int* __restrict__ slots,
                                  T* __restrict__ keys, T* __restrict__ values, int q_heads, int kv_heads,
                                  int head_dim, int rot, int page_size, int write_cache,
                                  const float* __restrict__ partial, int splits, size_t split_stride,
                                  const float* __restrict__ bias, int adjacent) {
  const int head = blockIdx.x, n = blockIdx.y;
  const int width = (q_heads + 2 * kv_heads) * head_dim;
  const int half = rot / 2;
  const int col0 = head * head_dim;
  const float* src = partial + (size_t)n * width + col0;
  // The sums of two columns at once, every load issued before the first is waited for (the
  // kernel's time is a chain of memory latencies); added in split order, then the bias.
  auto values2 = [&](int d0, int d1, float& v0, float& v1) {
    v0 = 0.f;
    v1 = 0.f;
    const float b0 = bias ? bias[col0 + d0] : 0.f, b1 = bias ? bias[col0 + d1] : 0.f;
    for (int s0 = 0; s0 < splits; s0 += 8) {
      float a0[8], a1[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        a0[i] = s0 + i < splits ? src[(s0 + i) * split_stride + d0] : 0.f;
        a1[i] = s0 + i < splits ? src[(s0 + i) * split_stride + d1] : 0.f;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (s0 + i < splits) {
          v0 += a0[i];
          v1 += a1[i];
        }
    }
    if (bias) {
      v0 += b0;
      v1 += b1;
    }
    v0 = tw_to_float(tw_from_float<T>(v0));           // what the projection would have stored
    v1 = tw_to_float(tw_from_float<T>(v1));
  };
  const int slot = write_cache ? slots[n] : -1;
  const int page = slot >= 0 ? slot / page_size : 0;
  const int off = slot >= 0 ? slot % page_size : 0;
  T* row = qkv + (size_t)n * ld + col0;
  if (head < q_heads + kv_heads) {
    const bool is_q = head < q_heads;
    if (!is_q && slot < 0) return;
    T* dst = is_q ? row : keys + (((size_t)page * kv_heads + (head - q_heads)) * page_size + off) * head_dim;
    for (int j = threadIdx.x; j < half; j += blockDim.x) {
      const float cj = cos_t[(size_t)n * half + j], sj = sin_t[(size_t)n * half + j];
      const int i_lo = adjacent ? 2 * j : j, i_hi = adjacent ? 2 * j + 1 : j + half;
      float lo, hi;
      values2(i_lo, i_hi, lo, hi);
      float r_lo, r_hi;
      tw_rotate_pair(lo, hi, cj, sj, r_lo, r_hi);
      dst[i_lo] = tw_from_float<T>(r_lo);
      dst[i_hi] = tw_from_float<T>(r_hi);
    }
    for (int d = rot + threadIdx.x; d < head_dim; d += 2 * blockDim.x) {      // the part that is not rotated
      const int d1 = d + blockDim.x < head_dim ? d + blockDim.x : d;
      float v0, v1;
      values2(d, d1, v0, v1);
      dst[d] = tw_from_float<T>(v0);
      if (d1 != d) dst[d1] = tw_from_float<T>(v1);
    }
  } else {
    if (slot < 0) return;
    const int kh = head - q_heads - kv_heads;
    T* dst = values + ((size_t)page * kv_heads + kh) * head_dim * page_size + off;
    for (int d = threadIdx.x; d < head_dim; d += 2 * blockDim.x) {
      const int d1 = d + blockDim.x < head_dim ? d + blockDim.x : d;
      float v0, v1;
      values2(d, d1, v0, v1);
      dst[(size_t)d * page_size] = tw_from_float<T>(v0);
      if (d1 != d) dst[(size_t)d1 * page_size] = tw_from_float<T>(v1);
    }
  }
}

extern "C" int tw_rope_kv_write(int dtype, void* qkv, long ld, const float* cos_t, const float* sin_t,
                                const int* slots, void* keys, void* values, int n, int q_heads,
                                int kv_heads, int head_dim, int rot, int page_size, int write_cache,
                                const float* partial, int splits, const float* bias, int adjacent,
                                hipStream_t stream) {
  TW_REQUIRE(partial == nullptr || splits >= 1);
  const size_t split_stride = (size_t)n * (q_heads + 2 * kv_heads) * head_dim;
  TW_REQUIRE(n >= 0 && q_heads > 0 && kv_heads > 0 && head_dim > 0 && page_size > 0);
  TW_REQUIRE(rot >= 0 && rot <= head_dim && rot % 2 == 0);
  TW_REQUIRE(ld >= (long)(q_heads + 2 * kv_heads) * head_dim);
  TW_REQUIRE(!write_cache || (slots && keys && values));
  if (n == 0) return 0;
  if (partial) {
    TW_REQUIRE(n <= 65535);
    dim3 grid(q_heads + 2 * kv_heads, n);
    const int threads = head_dim / 2 <= 64 ? 64 : 128;
    if (dtype == TW_DTYPE_F32)
      qkv_finish_kernel<float><<<grid, threads, 0, stream>>>((float*)qkv, ld, cos_t, sin_t, slots, (float*)keys,
                                                            (float*)values, q_heads, kv_heads, head_dim, rot,
                                                            page_size, write_cache, partial, splits, split_stride, bias, adjacent);
    else if (dtype == TW_DTYPE_BF16)
      qkv_finish_kernel<bf16_t><<<grid, threads, 0, stream>>>((bf16_t*)qkv, ld, cos_t, sin_t, slots, (bf16_t*)keys,
                                                             (bf16_t*)values, q_heads, kv_heads, head_dim, rot,
                                                             page_size, write_cache, partial, splits, split_stride, bias, adjacent);
    else
      return TW_ERR_BAD_ARGUMENT;
    return TW_LAUNCH_RESULT();
  }
  // the whole head rotated in halves, everything 16-byte aligned: the vector form
  const int per16 = dtype == TW_DTYPE_F32 ? 4 : 8;
  if (rot == head_dim && !adjacent && head_dim % (2 * per16) == 0 && ld % per16 == 0 &&
      (uintptr_t)qkv % 16 == 0 && (uintptr_t)cos_t % 16 == 0 && (uintptr_t)sin_t % 16 == 0 &&
      (!write_cache || ((uintptr_t)keys % 16 == 0 && (uintptr_t)values % 16 == 0))) {
    if (dtype == TW_DTYPE_F32)
      rope_kv_write_vec_kernel<float><<<n, 256, 0, stream>>>((float*)qkv, ld, cos_t, sin_t, slots, (float*)keys,
                                                             (float*)values, q_heads, kv_heads, head_dim,
                                                             page_size, write_cache);
    else if (dtype == TW_DTYPE_BF16)
      rope_kv_write_vec_kernel<bf16_t><<<n, 256, 0, stream>>>((bf16_t*)qkv, ld, cos_t, sin_t, slots, (bf16_t*)keys,
                                                              (bf16_t*)values, q_heads, kv_heads, head_dim,
                                                              page_size, write_cache);
    else
      return TW_ERR_BAD_ARGUMENT;
    return TW_LAUNCH_RESULT();
  }
  if (dtype == TW_DTYPE_F32)
    rope_kv_write_kernel<float><<<n, 256, 0, stream>>>((float*)qkv, ld, cos_t, sin_t, slots, (float*)keys,
                                                       (float*)values, q_heads, kv_heads, head_dim, rot,
                                                       page_size, write_cache, adjacent);
  else if (dtype == TW_DTYPE_BF16)
    rope_kv_write_kernel<bf16_t><<<n, 256, 0, stream>>>((bf16_t*)qkv, ld, cos_t, sin_t, slots,
                                                        (bf16_t*)keys, (bf16_t*)values, q_heads, kv_heads,
                                                        head_dim, rot, page_size, write_cache, adjacent);
  else
    return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}

// ---- SiLU-multiply: out[n, i] = silu(gu[n, i]) * gu[n, inter + i] -------------------------------
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, long n, int inter) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n * inter) return;
  const long row = i / inter;
  const int col = (int)(i % inter);
  const float g = tw_to_float(gu[row * 2 * inter + col]);
  const float u = tw_to_float(gu[row * 2 * inter + inter + col]);
  out[i] = tw_from_float<T>(g / (1.0f + expf(-g)) * u);
}

extern "C" int tw_silu_mul(int dtype, const void* gu, void* out, int n, int inter, hipStream_t stream) {
  TW_REQUIRE(n >= 0 && inter > 0);
  if (n == 0) return 0;
  const int blocks = tw_div_up((long)n * inter, 256);
  if (dtype == TW_DTYPE_F32)
    silu_mul_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gu, (float*)out, n, inter);
  else if (dtype == TW_DTYPE_BF16)
    silu_mul_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, n, inter);
  else
    return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}
