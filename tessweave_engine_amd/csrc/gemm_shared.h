// Shared by the two linear-layer sources: gemm.hip (few rows, any K, the C entry points) and
// gemm_tiled.hip (many rows), which are compiled apart because they want different register
// allocation for their MFMA accumulators.
#pragma once
#include "tw_common.h"

__device__ __forceinline__ float tw_silu(float g) { return g / (1.0f + expf(-g)); }

// Sum of split-K partial sums partial[split][M][N], in split order, then bias and residual.
template <typename OutT>
__global__ void splitk_reduce_kernel(const float* __restrict__ partial, int splits,
                                     const float* __restrict__ bias, const float* residual, long ldr,
                                     OutT* C, long ldc, int M, int N) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long)M * N) return;
  const int row = (int)(i / N), col = (int)(i % N);
  float v = 0.f;
  for (int s = 0; s < splits; ++s) v += partial[(size_t)s * M * N + i];
  if (bias) v += bias[col];
  if (residual) v += residual[(size_t)row * ldr + col];
  C[(size_t)row * ldc + col] = tw_from_float<OutT>(v);
}

// The same sums, four columns per thread with 16-byte loads and stores (N, the leading dimensions
// and the pointers allow it): every element is still added in the order above, so the two kernels
// give the same bits. All the loads of a thread are issued before the first addition.
template <typename OutT>
__global__ void splitk_reduce_vec4_kernel(const float* __restrict__ partial, int splits,
                                          const float* __restrict__ bias, const float* residual, long ldr,
                                          OutT* C, long ldc, int M, int N) {
  const long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i >= (long)M * N) return;
  const int row = (int)(i / N), col = (int)(i % N);
  const size_t plane = (size_t)M * N;
  f32x4 v = {0.f, 0.f, 0.f, 0.f};
  const f32x4 b = bias ? *reinterpret_cast<const f32x4*>(bias + col) : f32x4{0.f, 0.f, 0.f, 0.f};
  const f32x4 r = residual ? *reinterpret_cast<const f32x4*>(residual + (size_t)row * ldr + col) : f32x4{0.f, 0.f, 0.f, 0.f};
  for (int s0 = 0; s0 < splits; s0 += 4) {
    f32x4 a[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
      a[k] = s0 + k < splits ? *reinterpret_cast<const f32x4*>(partial + (size_t)(s0 + k) * plane + i) : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (s0 + k < splits) v = v + a[k];
  }
  if (bias) v = v + b;
  if (residual) v = v + r;
  OutT* dst = C + (size_t)row * ldc + col;
  if (sizeof(OutT) == 4) {
    *reinterpret_cast<f32x4*>(dst) = v;
  } else {
    OutT packed[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) packed[e] = tw_from_float<OutT>(v[e]);
    *reinterpret_cast<uint64_t*>(dst) = *reinterpret_cast<const uint64_t*>(packed);
  }
}

template <typename OutT>
static inline int launch_splitk_reduce(const float* partial, int splits, const float* bias, const float* residual,
                                       long ldr, OutT* C, long ldc, int M, int N, hipStream_t stream) {
  const bool vec = N % 4 == 0 && ldc % 4 == 0 && (residual == nullptr || ldr % 4 == 0) &&
                   (uintptr_t)partial % 16 == 0 && (uintptr_t)C % (4 * sizeof(OutT)) == 0 &&
                   (bias == nullptr || (uintptr_t)bias % 16 == 0) && (residual == nullptr || (uintptr_t)residual % 16 == 0);
  if (vec)
    splitk_reduce_vec4_kernel<OutT><<<tw_div_up((long)M * N / 4, 256), 256, 0, stream>>>(partial, splits, bias, residual,
                                                                                       ldr, C, ldc, M, N);
  else
    splitk_reduce_kernel<OutT><<<tw_div_up((long)M * N, 256), 256, 0, stream>>>(partial, splits, bias, residual, ldr, C,
                                                                              ldc, M, N);
  return TW_LAUNCH_RESULT();
}

// The tiled kernels (gemm_tiled.hip). shape: 0 = choose, 1 = tiles of 128x128, 2 = 128x256,
// 3 = 256x256 (bfloat16 with shuffled weights only). Returns 0 or an error code.
int tw_tiled_linear(int dtype, int out_f32, int shuffled, int glu, int shape, const void* A, long lda,
                    const void* W, long ldw, const float* bias, const float* residual, long ldr, void* C,
                    long ldc, float* partial, long partial_bytes, int M, int N, int K, hipStream_t stream);
// The tiled kernels with the sums of their K ranges left in partial[s][M][N] (no reduction kernel), and
// the number of ranges they would use (1: none; then partial[0] is the product).
int tw_tiled_partial_splits(int dtype, int shuffled, long lda, int M, int N, int K);
int tw_tiled_partials(int dtype, int shuffled, const void* A, long lda, const void* W, long ldw, float* partial,
                      long partial_bytes, int M, int N, int K, int* splits_used, hipStream_t stream);
// Bytes of split-K scratch the tiled kernels can use for `rows` rows of an [N, K] weight (0: none).
long tw_tiled_workspace_bytes(int dtype, int rows, int N, int K);
